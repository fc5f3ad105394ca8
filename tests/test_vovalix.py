"""Vovalix without a GPU: configuration, registry, the schedule of layers that borrow tensors,
the checkpoint layout, sizes taken from tensor shapes, and the plain implementation's own
consistency."""

from __future__ import annotations

import copy

import pytest
import torch

from tests.plain import vovalix as plain
from tests.vovalix_helpers import CONFIG_A, CONFIG_B, CONFIG_C, CONFIGS


def spec_of(config):
    from kvcore_amd.registry import resolve_architecture

    arch = resolve_architecture(config)
    return arch.build_spec(arch.parse_config(config))


def test_the_architecture_is_registered_with_a_way_to_complete_its_configuration():
    from kvcore_amd.registry import resolve_architecture

    arch = resolve_architecture(CONFIG_A)
    assert arch.name == "Vovalix" and arch.complete_config is not None


def test_a_layer_that_borrows_tensors_is_a_second_run_of_its_owner():
    from kvcore_amd.models.decoder import DecoderModel

    spec = spec_of(CONFIG_A)
    assert len(spec.layers) == 4  # five layers, one of them borrowed
    assert [e.layer for e in spec.resolved_schedule()] == [0, 1, 2, 1, 3]
    assert [l.prefix for l in spec.layers] == ["l0", "l1", "l2", "l4"]
    model = DecoderModel(spec, torch.float32, "cpu")
    # two attention layers of different sizes: two cache groups of one plane each
    assert sorted(g.num_planes for g in model.cache_groups) == [1, 1]
    # every run has states of its own: gla one array, delta two (convolution inputs, matrices)
    per_call = [len(c.state_indices) for c in model.calls]
    assert per_call == [0, 1, 2, 1, 0]
    seen = [i for c in model.calls for i in c.state_indices]
    assert seen == list(range(len(model.state_arrays)))
    shapes = [tuple(model.state_arrays[i].need.shape) for i in seen]
    assert shapes == [(3, 24, 40), (2, 2 * 2 * 24 + 4 * 20), (4, 24, 20), (3, 24, 40)]
    spec_b = spec_of(CONFIG_B)
    assert [e.layer for e in spec_b.resolved_schedule()] == [0, 1, 2, 1]
    model_b = DecoderModel(spec_b, torch.float32, "cpu")
    assert [g.num_planes for g in model_b.cache_groups] == [2]  # the borrowed attention layer's own plane


def test_checkpoint_layout_has_the_design_s_names_and_shapes():
    from kvcore_amd.weights.loader import checkpoint_layout

    layout = {k: v[0] for k, v in checkpoint_layout(spec_of(CONFIG_A)).items()}
    assert layout["embed"] == (211, 96) and "head" not in layout and "head.weight" not in layout
    assert layout["final.norm"] == (96,) and layout["l0.norm1"] == (96,)
    assert layout["l0.mix.q"] == (128, 96) and layout["l0.mix.k"] == (64, 96) and layout["l0.mix.v"] == (32, 96)
    assert layout["l0.mix.o"] == (96, 64)
    assert layout["l1.mix.a1"] == (12, 96) and layout["l1.mix.a2"] == (72, 12) and layout["l1.mix.a2.b"] == (72,)
    assert layout["l1.mix.norm"] == (40,) and layout["l1.mix.g"] == (120, 96)
    assert layout["l2.mix.q.conv"] == (48, 3) and layout["l2.mix.v.conv"] == (80, 3)
    assert layout["l2.mix.b"] == (4, 96) and layout["l2.mix.A_log"] == (4,) and layout["l2.mix.dt_bias"] == (4,)
    assert layout["l0.mlp.router"] == (6, 96) and layout["l0.mlp.e5.gate"] == (40, 96)
    assert layout["l0.mlp.e0.down"] == (96, 40) and layout["l0.mlp.shared.up"] == (56, 96)
    assert not any(k.startswith("l3.") for k in layout)  # the borrowed layer has no tensors
    assert not any(k.startswith("l4.mlp") for k in layout)  # a layer without a feed-forward
    assert not any("shared" in k for k in checkpoint_layout(spec_of(CONFIG_B)) if k.startswith("l0."))


def test_the_decay_rank_comes_from_a_tensor_s_shape_when_the_file_leaves_it_out():
    from kvcore_amd.config.model_config import ConfigError
    from kvcore_amd.registry import resolve_architecture

    arch = resolve_architecture(CONFIG_A)
    bare = copy.deepcopy(CONFIG_A)
    for layer in bare["layers"]:
        layer["mixer"].pop("rank", None)
    with pytest.raises(ConfigError, match="rank"):
        arch.parse_config(bare)
    filled = arch.complete_config(bare, {"l1.mix.a1": (7, 96)}.get)
    typed = arch.parse_config(filled)
    assert typed.layers[1].mixer.rank == 7 and typed.layers[3].mixer.rank == 7
    assert arch.parse_config(arch.complete_config(CONFIG_A, {"l1.mix.a1": (7, 96)}.get)).layers[1].mixer.rank == 12


def test_configuration_errors_name_the_key():
    from kvcore_amd.config.model_config import ConfigError
    from kvcore_amd.config.vovalix_config import VovalixConfig

    for path, value, word in ((("layers", 0, "type"), "mamba", "type"), (("layers", 0, "mixer", "kv_heads"), 3, "kv_heads"),
                              (("layers", 0, "mlp", "router", "groups", "count"), 4, "router"),
                              (("layers", 3, "weights_of"), 4, "weights_of"), (("norm",), None, "norm")):
        bad = copy.deepcopy(CONFIG_A)
        at = bad
        for key in path[:-1]:
            at = at[key]
        at[path[-1]] = value
        with pytest.raises(ConfigError, match=word):
            VovalixConfig.from_dict(bad)
    typed = VovalixConfig.from_dict(CONFIG_C)
    assert typed.logit_scale == 1.0 and typed.layers[3].mixer.chunk == 0 and typed.layers[1].mixer.chunk == 1
    assert typed.layers[3].mlp.groups == 1 and typed.layers[0].mlp.shared_ff == 0


def test_distance_slopes_and_constants_of_the_design():
    from kvcore_amd.models.vovalix import distance_slopes

    assert distance_slopes(8) == tuple(plain.distance_slopes(8))
    assert distance_slopes(1) == (2.0 ** -8,) and abs(distance_slopes(4)[0] - 0.25) < 1e-12


def _random_weights(config, seed):
    from kvcore_amd.weights.loader import checkpoint_layout

    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, (shape, _, _) in checkpoint_layout(spec_of(config)).items():
        out[name] = torch.randn(shape, generator=gen, dtype=torch.float64) * (0.2 if len(shape) == 2 else 0.5)
    return out


@pytest.mark.parametrize("name", list(CONFIGS))
def test_plain_model_is_causal_and_its_recurrences_carry_over(name):
    """A prefix's logits do not change when tokens follow, for every configuration."""
    config = CONFIGS[name][0]
    w = _random_weights(config, 3)
    gen = torch.Generator().manual_seed(5)
    tokens = torch.randint(0, config["vocab"], (37,), generator=gen).tolist()
    full, layers = plain.vovalix_forward(config, w, tokens, return_layers=True)
    assert layers.shape == (len(config["layers"]), 37, config["width"])
    part = plain.vovalix_forward(config, w, tokens[:20])
    assert torch.allclose(full[:20], part, atol=1e-9, rtol=1e-9)


def test_plain_recurrences_against_their_closed_forms():
    gen = torch.Generator().manual_seed(1)
    T, d, dv = 9, 4, 3
    q, k, a = (torch.rand(T, d, generator=gen, dtype=torch.float64) for _ in range(3))
    v = torch.randn(T, dv, generator=gen, dtype=torch.float64)
    o = plain.gated_linear_recurrence(q, k, v, a)
    # o_t = sum_(j<=t) (q_t * prod_(j<i<=t) a_i) . k_j  v_j
    for t in (0, 4, 8):
        want = torch.zeros(dv, dtype=torch.float64)
        for j in range(t + 1):
            want += ((q[t] * a[j + 1:t + 1].prod(dim=0)) @ k[j]) * v[j]
        assert torch.allclose(o[t], want, atol=1e-12)
    # the delta rule with beta = 1, g = 1 and orthonormal keys stores each value exactly
    keys = torch.eye(d, dtype=torch.float64)
    vals = torch.randn(d, dv, generator=gen, dtype=torch.float64)
    o = plain.delta_recurrence(keys, keys, vals, torch.ones(d, dtype=torch.float64), torch.ones(d, dtype=torch.float64))
    assert torch.allclose(o, vals, atol=1e-12)
    # and a key written twice is overwritten, not added to
    k2 = torch.stack([keys[0], keys[0]])
    o = plain.delta_recurrence(k2, k2, vals[:2], torch.ones(2, dtype=torch.float64), torch.ones(2, dtype=torch.float64))
    assert torch.allclose(o[1], vals[1], atol=1e-12)


def test_plain_routing_keeps_to_the_best_groups():
    s = torch.tensor([0.05, 0.30, 0.02, 0.03, 0.25, 0.20, 0.10, 0.05], dtype=torch.float64)
    chosen, w = plain.route(s, top=3, groups=4, keep=2)  # groups (0,1) (2,3) (4,5) (6,7): best are 0 and 2
    assert chosen == [1, 4, 5] and abs(float(w.sum()) - 1.0) < 1e-12
    chosen, _ = plain.route(s, top=3, groups=1, keep=1)
    assert chosen == [1, 4, 5]
    chosen, _ = plain.route(s, top=2, groups=4, keep=1)
    assert chosen == [1, 0]
    chosen, _ = plain.route(torch.tensor([0.25, 0.25, 0.25, 0.25], dtype=torch.float64), top=2, groups=2, keep=1)
    assert chosen == [0, 1]  # ties go to the lower index


def test_plain_chunked_attention_sees_its_own_chunk_only():
    gen = torch.Generator().manual_seed(2)
    T, d = 12, 8
    q = torch.randn(T, 2, d, generator=gen, dtype=torch.float64)
    k = torch.randn(T, 1, d, generator=gen, dtype=torch.float64)
    v = torch.randn(T, 1, 3, generator=gen, dtype=torch.float64)
    o = plain.chunked_distance_attention(q, k, v, 0.3, 5, 1e-6)
    assert torch.allclose(o[5], v[5].expand(2, 3)) and torch.allclose(o[10], v[10].expand(2, 3))
    v2 = v.clone()
    v2[:5] += 1.0  # tokens of the first chunk do not matter to the second
    o2 = plain.chunked_distance_attention(q, k, v2, 0.3, 5, 1e-6)
    assert torch.allclose(o[5:], o2[5:]) and not torch.allclose(o[:5], o2[:5])
