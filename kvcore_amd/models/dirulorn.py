"""The Dirulorn decoder as a ``ModelSpec``.

Pre-norm layers with layer norms (weight and bias) on a float32 stream.  A layer's mixer is
either a state-space mixer (``mamba2``) or two mixers side by side (``parallel``): grouped-query
attention whose keys and values differ in size, with a norm of every query and key head and a
partial interleaved rotation, beside a gated linear recurrent block; each branch is divided by
its root mean square and the two are averaged.  A stretch of layers may run several times with
the same weights: every pass has caches and states of its own (one schedule entry a run) and is
opened by a product over the stream and the embedding's output side by side, plus a vector of
the pass.  Tensor names: ``embed``, ``head``, ``final.norm[.b]``, ``loop.in``, ``loop.step``,
``l<i>.norm1[.b]``, ``l<i>.norm2[.b]``, ``l<i>.mix.*``, ``l<i>.mlp.{gate,up,down}``.
"""

from __future__ import annotations

from kvcore_amd.config.dirulorn_config import DirulornConfig, ParallelMixerConfig, StateSpaceConfig
from kvcore_amd.parts.base import PartSpec

from .spec import LayerSpec, ModelSpec, ScheduleEntry

DECAY_SCALE = 8.0  # the recurrent unit's log a = -DECAY_SCALE * r * softplus(lam)


def dirulorn_spec(config: DirulornConfig) -> ModelSpec:
    H, eps = config.width, config.eps

    def norm() -> PartSpec:
        return PartSpec("layernorm", {"hidden_size": H, "eps": eps, "weight_name": "", "bias_name": "b"})

    positions: list[PartSpec] = []

    def position_of(rot) -> int | None:
        if rot is None:
            return None
        scaling = None
        if rot.scaling is not None:
            factor, low, high, original = rot.scaling
            scaling = {"rope_type": "llama3", "factor": factor, "low_freq_factor": low,
                       "high_freq_factor": high, "original_max_position_embeddings": original}
        spec = PartSpec("rotary", {"rot_dim": rot.dims, "theta": rot.base, "scaling": scaling,
                                   "interleaved": True})
        if spec not in positions:
            positions.append(spec)
        return positions.index(spec)

    layers = []
    for i, layer in enumerate(config.layers):
        position = None
        m = layer.mixer
        if isinstance(m, StateSpaceConfig):
            mixer = PartSpec("state_space", {
                "hidden_size": H, "heads": m.heads, "head_dim": m.vdim, "state_size": m.state,
                "groups": m.groups, "conv": m.conv, "norm_groups": m.norm_groups, "eps": eps,
                "tensor_names": {"in": "in", "conv": "conv", "conv_bias": "conv.b", "dt_bias": "dt_bias",
                                 "a_log": "A_log", "d": "D", "norm": "norm", "o": "o"}})
        else:
            assert isinstance(m, ParallelMixerConfig)
            left, right = m.left, m.right
            position = position_of(left.rot)
            attention = PartSpec("paged_attention", {
                "hidden_size": H, "num_heads": left.heads, "num_kv_heads": left.kv_heads,
                "head_dim": left.dim, "v_head_dim": left.vdim, "scale": left.scale, "qk_norm_eps": eps,
                "tensor_names": {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm"}})
            recurrent = PartSpec("gated_linear_recurrence", {
                "hidden_size": H, "width": right.width, "blocks": right.blocks, "conv": right.conv,
                "decay_scale": DECAY_SCALE,
                "tensor_names": {"y": "y", "y_bias": "y.b", "x": "x", "x_bias": "x.b", "conv": "conv",
                                 "conv_bias": "conv.b", "gate_a": "ra", "gate_a_bias": "ra.b",
                                 "gate_i": "ri", "gate_i_bias": "ri.b", "lam": "lam", "o": "o"}})
            mixer = PartSpec("parallel", {"hidden_size": H, "eps": eps, "gain_suffix": ".out",
                                          "branches": (("left", attention), ("right", recurrent))})
        norms = {"norm1": norm()}
        if layer.ff is None:
            ffn = PartSpec("none")
        else:
            norms["norm2"] = norm()
            ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": layer.ff, "gate_name": "gate",
                                      "up_name": "up", "down_name": "down", "suffix": "",
                                      "sized_buffers": True})
        layers.append(LayerSpec(
            prefix=f"l{i}", mixer=mixer, ffn=ffn, norms=norms,
            block=PartSpec("prenorm", {"mixer_name": "mix", "ffn_name": "mlp", "input_norm": "norm1",
                                       "post_norm": None if layer.ff is None else "norm2"}),
            position=position))

    n = len(layers)
    schedule: tuple[ScheduleEntry, ...] = ()
    stream_ops: tuple[PartSpec, ...] = ()
    if config.loop is not None:
        lp = config.loop
        entries = [ScheduleEntry(i) for i in range(lp.start)]
        for t in range(lp.times):
            for i in range(lp.start, lp.stop):
                entries.append(ScheduleEntry(i, before=0 if i == lp.start else None, before_arg=t))
        entries += [ScheduleEntry(i) for i in range(lp.stop, n)]
        schedule = tuple(entries)
        stream_ops = (PartSpec("loop_inject", {"hidden_size": H, "passes": lp.times,
                                               "weight_name": "in", "step_name": "step"}),)
    return ModelSpec(
        vocab_size=config.vocab, hidden_size=H, max_position_embeddings=config.max_position_embeddings,
        layers=tuple(layers), final_norm=norm(), positions=tuple(positions), schedule=schedule,
        stream_ops=stream_ops, stream_op_prefixes=("loop",) if stream_ops else (),
        embedding=PartSpec("token_embedding", {"vocab_size": config.vocab, "hidden_size": H, "weight_name": ""}),
        head=PartSpec("linear_head", {"vocab_size": config.vocab, "hidden_size": H, "weight_name": ""}),
        eos_token_ids=config.eos_token_ids, embed_prefix="embed", final_norm_prefix="final.norm",
        head_prefix="head", ignored_suffixes=(),
    )
