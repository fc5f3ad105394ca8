"""Dirulorn without a GPU: configuration, registry, the schedule of a looped model, the
checkpoint layout, and the plain implementation's own consistency."""

from __future__ import annotations

import copy

import pytest
import torch

from tests.dirulorn_helpers import CONFIG_P, CONFIG_Q, CONFIG_R, CONFIGS
from tests.plain import dirulorn as plain


def spec_of(config):
    from kvcore_amd.registry import resolve_architecture

    arch = resolve_architecture(config)
    return arch.build_spec(arch.parse_config(config))


def test_the_architecture_is_found_by_its_name_in_the_singular():
    from kvcore_amd.registry import resolve_architecture

    assert resolve_architecture(CONFIG_P).name == "Dirulorn"
    assert resolve_architecture({"architectures": ["Dirulorn"]}).name == "Dirulorn"


def test_schedule_of_a_loop_names_a_pass_opener_per_pass():
    spec = spec_of(CONFIG_P)  # layers 1..2 three times
    runs = [(e.layer, e.before, e.before_arg if e.before is not None else None) for e in spec.resolved_schedule()]
    assert runs == [(0, None, None), (1, 0, 0), (2, None, None), (1, 0, 1), (2, None, None), (1, 0, 2),
                    (2, None, None), (3, None, None)]
    assert [r[0] for r in runs] == [i for i, _ in plain.layer_runs(CONFIG_P)]
    assert spec_of(CONFIG_Q).stream_ops == () and len(spec_of(CONFIG_Q).resolved_schedule()) == 3
    whole = spec_of(CONFIG_R)
    assert [e.layer for e in whole.resolved_schedule()] == [0, 1, 2, 0, 1, 2]


def test_every_run_of_a_looped_layer_has_cache_and_states_of_its_own():
    from kvcore_amd.models.decoder import DecoderModel

    model = DecoderModel(spec_of(CONFIG_P), torch.float32, "cpu")
    calls = model.calls
    assert len(calls) == 8
    # the attention of layers 0 and 2 differ in size: two cache groups; layer 2 runs three times
    assert len(model.cache_groups) == 2
    assert sorted(g.num_planes for g in model.cache_groups) == [1, 3]
    seen = [i for c in calls for i in c.state_indices]
    assert seen == list(range(len(model.state_arrays))) and len(seen) == 2 * 8
    assert model.cache_groups[0].need.planes == ((2, 32), (2, 16))


def test_checkpoint_layout_has_the_design_s_names_and_shapes():
    from kvcore_amd.weights.loader import checkpoint_layout

    layout = {k: v[0] for k, v in checkpoint_layout(spec_of(CONFIG_P)).items()}
    assert layout["embed"] == (211, 96) and layout["head"] == (211, 96)
    assert layout["final.norm"] == (96,) and layout["final.norm.b"] == (96,)
    assert layout["loop.in"] == (96, 192) and layout["loop.step"] == (3, 96)
    assert layout["l0.mix.left.q"] == (128, 96) and layout["l0.mix.left.v"] == (32, 96)
    assert layout["l0.mix.left.q.norm"] == (32,) and layout["l0.mix.left.o"] == (96, 64)
    assert layout["l0.mix.right.ra"] == (3, 24, 24) and layout["l0.mix.right.conv"] == (72, 3)
    assert layout["l0.mix.left.out"] == (96,) and layout["l0.mix.right.out"] == (96,)
    assert layout["l1.mix.in"] == (2 * 120 + 2 * 3 * 24 + 6, 96) and layout["l1.mix.conv"] == (120 + 144, 3)
    assert layout["l1.mix.A_log"] == (6,) and layout["l1.mix.norm"] == (120,)
    assert "l1.norm2" not in layout and "l1.mlp.gate" not in layout  # a layer without a feed-forward
    assert layout["l3.mlp.down"] == (96, 200) and layout["l3.norm2.b"] == (96,)
    assert "loop.in" not in checkpoint_layout(spec_of(CONFIG_Q))


@pytest.mark.parametrize("change,match", [
    (lambda c: c["layers"][0].update(type="window"), "not supported"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "not supported"),
    (lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][1]["mixer"].update(groups=4), "fit together"),
    (lambda c: c["loop"].update(stop=9), "does not fit"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=34), "rot.dims"),
])
def test_configurations_that_do_not_fit_are_refused_by_name(change, match):
    from kvcore_amd.config.model_config import ConfigError

    config = copy.deepcopy(CONFIG_P)
    change(config)
    with pytest.raises(ConfigError, match=match):
        spec_of(config)


@pytest.mark.parametrize("name", list(CONFIGS))
def test_the_plain_model_is_causal_and_its_loop_changes_the_result(name, tmp_path):
    """Logits at a position do not change when tokens are appended; a model with one pass
    fewer gives other logits (the passes are really run)."""
    config = CONFIGS[name][0]
    gen = torch.Generator().manual_seed(3)
    from kvcore_amd.weights.loader import checkpoint_layout

    w = {k: torch.randn(shape, generator=gen, dtype=torch.float64) * 0.2
         for k, (shape, _, _) in checkpoint_layout(spec_of(config)).items()}
    tokens = [int(t) for t in torch.randint(0, config["vocab"], (12,), generator=gen)]
    full = plain.forward(config, w, tokens)
    assert torch.allclose(plain.forward(config, w, tokens[:7]), full[:7], atol=1e-12)
    if config.get("loop") and config["loop"]["times"] > 1:
        fewer = copy.deepcopy(config)
        fewer["loop"]["times"] -= 1
        assert not torch.allclose(plain.forward(fewer, w, tokens), full, atol=1e-6)


def test_rotary_frequencies_keep_slow_and_blend():
    f = plain.rotary_frequencies(8, 100.0, {"factor": 4.0, "low": 1.0, "high": 2.0, "original": 24})
    base = [100.0 ** (-2 * i / 8) for i in range(4)]
    assert f[0] == base[0]                      # wavelength 6.3 < 12: kept
    assert abs(f[3] - base[3] / 4.0) < 1e-15    # wavelength 199 > 24: slowed
    assert base[1] / 4.0 < f[1] < base[1]       # wavelength 19.9: between
    from kvcore_amd.parts.rotary import rotary_inv_freq

    got = rotary_inv_freq(8, 100.0, {"rope_type": "llama3", "factor": 4.0, "low_freq_factor": 1.0,
                                     "high_freq_factor": 2.0, "original_max_position_embeddings": 24})
    assert torch.allclose(got.double(), torch.tensor(f, dtype=torch.float64), rtol=1e-6)
