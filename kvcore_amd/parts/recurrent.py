"""Mixers that carry a state of fixed size per request instead of a cache that grows.

``GatedLinearRecurrence`` is the recurrent block of Griffin: two branches of the same width,
``y = gelu_tanh(W_y h + b_y)`` and ``u = conv(W_x h + b_x)`` (a short causal convolution per
channel), a real-gated linear recurrent unit on ``u`` whose gates are block-diagonal,

    r = sigmoid(A_b u_b + a_b),  i = sigmoid(I_b u_b + i_b),
    a = exp(-c r softplus(lam)),  S_t = a S_(t-1) + sqrt(1 - a^2) i u,

and the output ``W_o (S * y)``.

``StateSpaceMixer`` is Mamba-2's mixer: one input product laid out ``[z | x | B | C | dt]``; x,
B and C pass a short causal convolution and silu; per head, with a scalar decay,

    dt = softplus(dt + dt_bias),  S_t = exp(-exp(A_log) dt) S_(t-1) + dt B_t x_t^T,
    y_t = S_t^T C_t + D x_t;

then ``y * silu(z)``, an RMS norm in equal parts of the width, and the output product.

Both keep their recurrent state and the last ``taps - 1`` inputs of their convolution in
float32 slot arrays; a request starts from zeros at position 0.  Everything that enters a
recurrence (decays, step sizes, gates, the convolution's results) is float32; the products
run in the model dtype with float32 sums.
"""

from __future__ import annotations

import torch

from kvcore_amd.ops import library as ops

from .base import Mixer, ParamSource, ParamSpec, StateNeed, register_mixer


def _src(name: str, rows: int) -> tuple[ParamSource, ...]:
    return (ParamSource(name, 0, rows),)


class GatedLinearRecurrence(Mixer):
    """``width`` channels in ``blocks`` equal parts for the gates, a convolution of ``conv``
    taps, decay constant ``decay_scale`` (the c above).  ``tensor_names`` renames checkpoint
    tensors (keys: y, y_bias, x, x_bias, conv, conv_bias, gate_a, gate_a_bias, gate_i,
    gate_i_bias, lam, o).  ``float32_result``: the output rows are float32 sums."""

    def __init__(self, *, hidden_size: int, width: int, blocks: int, conv: int,
                 decay_scale: float = 8.0, tensor_names: dict[str, str] | None = None,
                 float32_result: bool = False, position=None) -> None:
        if width <= 0 or blocks <= 0 or width % blocks:
            raise ValueError(f"{width} channels do not split into {blocks} equal blocks")
        if conv < 1:
            raise ValueError(f"a convolution needs at least one tap, got {conv}")
        self.hidden_size = hidden_size
        self.width = width
        self.blocks = blocks
        self.taps = conv
        self.decay_scale = float(decay_scale)
        self.float32_result = float32_result
        self.names = {"y": "y.weight", "y_bias": "y.bias", "x": "x.weight", "x_bias": "x.bias",
                      "conv": "conv.weight", "conv_bias": "conv.bias", "gate_a": "gate_a.weight",
                      "gate_a_bias": "gate_a.bias", "gate_i": "gate_i.weight",
                      "gate_i_bias": "gate_i.bias", "lam": "lam", "o": "o.weight",
                      **(tensor_names or {})}

    def param_specs(self) -> list[ParamSpec]:
        W, H, n, nb = self.width, self.hidden_size, self.names, self.blocks
        bw = W // nb
        return [
            ParamSpec("yx.weight", (2 * W, H),
                      sources=(ParamSource(n["y"], 0, W), ParamSource(n["x"], W, W))),
            ParamSpec("yx.bias", (2 * W,), init="zeros",
                      sources=(ParamSource(n["y_bias"], 0, W), ParamSource(n["x_bias"], W, W))),
            ParamSpec("conv.weight", (W, self.taps), kind="vector", init="normal", sources=_src(n["conv"], W)),
            ParamSpec("conv.bias", (W,), kind="vector", init="zeros", sources=_src(n["conv_bias"], W)),
            ParamSpec("gate_a.weight", (nb, bw, bw), kind="vector", init="normal", sources=_src(n["gate_a"], nb)),
            ParamSpec("gate_a.bias", (nb, bw), kind="vector", init="zeros", sources=_src(n["gate_a_bias"], nb)),
            ParamSpec("gate_i.weight", (nb, bw, bw), kind="vector", init="normal", sources=_src(n["gate_i"], nb)),
            ParamSpec("gate_i.bias", (nb, bw), kind="vector", init="zeros", sources=_src(n["gate_i_bias"], nb)),
            ParamSpec("lam", (W,), kind="vector", init="normal", sources=_src(n["lam"], W)),
            ParamSpec("o.weight", (H, W), sources=_src(n["o"], H)),
        ]

    def product_weights(self) -> tuple[str, ...]:
        return ("yx.weight", "o.weight")

    def state_needs(self) -> tuple[StateNeed, ...]:
        # the convolution's last inputs (at least one row, so that the array exists), the unit's state
        return (StateNeed((max(self.taps - 1, 1), self.width)), StateNeed((self.width,)))

    def forward(self, x, ctx, call, sink=None):
        p, W = self.params, self.width
        conv_state, lru_state = (ctx.states[i] for i in call.state_indices)
        conv_state = conv_state[:, : self.taps - 1]
        batch = dict(positions=ctx.positions, token_req=ctx.token_req, q_start=ctx.q_start,
                     slots=ctx.slots, num_reqs=ctx.num_reqs)
        yx = ctx.buf(f"lru_yx:{2 * W}", 2 * W)
        ops.linear(yx, x, p["yx.weight"], p["yx.bias"])
        u = ctx.buf(f"lru_u:{W}", W, torch.float32)
        ops.causal_conv(u, yx[:, W:], p["conv.weight"], p["conv.bias"], conv_state, act="none",
                        single_tokens=ctx.max_query_len == 1, **batch)
        a = ctx.buf(f"lru_a:{W}", W, torch.float32)
        drive = ctx.buf(f"lru_drive:{W}", W, torch.float32)
        ops.rglru_gates(a, drive, u, p["gate_a.weight"], p["gate_i.weight"], p["gate_a.bias"],
                        p["gate_i.bias"], p["lam"], self.decay_scale)
        gated = ctx.buf(f"lru_gated:{W}", W)
        # long portions are scanned in segments side by side, which takes a workspace
        need = ops.rglru_scan_workspace_floats(ctx.num_reqs, W, ctx.max_query_len)
        workspace = None
        if need:  # rows of 2 W sums; the buffer only ever grows, to the largest step seen
            workspace = ctx.buffers.get(f"lru_scan_sums:{W}", need // (2 * W), 2 * W, torch.float32,
                                        reserve=ctx.buffers.token_capacity // 32 + 2 * ctx.buffers.seq_capacity)
        ops.rglru_scan(gated, a, drive, yx[:, :W], lru_state, max_query_len=ctx.max_query_len,
                       workspace=workspace, **batch)
        if self.float32_result:
            out = ctx.buf("mixer_out_f32_b", self.hidden_size, torch.float32)
        else:
            out = ctx.buf("mixer_out", self.hidden_size)
        ops.linear(out, gated, p["o.weight"])
        return out


class StateSpaceMixer(Mixer):
    """``heads`` heads of ``head_dim`` value channels, a state of ``state_size`` rows a head, B
    and C shared by the heads of each of ``groups`` groups, a convolution of ``conv`` taps, the
    gated norm in ``norm_groups`` equal parts with ``eps``.  ``tensor_names`` renames checkpoint
    tensors (keys: in, conv, conv_bias, dt_bias, a_log, d, norm, o)."""

    def __init__(self, *, hidden_size: int, heads: int, head_dim: int, state_size: int, groups: int,
                 conv: int, norm_groups: int, eps: float, tensor_names: dict[str, str] | None = None,
                 position=None) -> None:
        if heads <= 0 or groups <= 0 or heads % groups:
            raise ValueError(f"{heads} heads do not split into {groups} groups")
        inner = heads * head_dim
        if norm_groups <= 0 or inner % norm_groups:
            raise ValueError(f"a width of {inner} does not split into {norm_groups} equal parts")
        if conv < 1:
            raise ValueError(f"a convolution needs at least one tap, got {conv}")
        self.hidden_size = hidden_size
        self.heads = heads
        self.head_dim = head_dim
        self.state_size = state_size
        self.groups = groups
        self.taps = conv
        self.norm_groups = norm_groups
        self.eps = eps
        self.inner = inner
        self.conv_dim = inner + 2 * groups * state_size
        self.proj_dim = inner + self.conv_dim + heads
        self.names = {"in": "in_proj.weight", "conv": "conv.weight", "conv_bias": "conv.bias",
                      "dt_bias": "dt_bias", "a_log": "A_log", "d": "D", "norm": "norm.weight",
                      "o": "out_proj.weight", **(tensor_names or {})}

    def param_specs(self) -> list[ParamSpec]:
        H, n, nh = self.hidden_size, self.names, self.heads
        return [
            ParamSpec("in_proj.weight", (self.proj_dim, H), sources=_src(n["in"], self.proj_dim)),
            ParamSpec("conv.weight", (self.conv_dim, self.taps), kind="vector", init="normal",
                      sources=_src(n["conv"], self.conv_dim)),
            ParamSpec("conv.bias", (self.conv_dim,), kind="vector", init="zeros",
                      sources=_src(n["conv_bias"], self.conv_dim)),
            ParamSpec("dt_bias", (nh,), kind="vector", init="normal", sources=_src(n["dt_bias"], nh)),
            ParamSpec("A_log", (nh,), kind="vector", init="normal", sources=_src(n["a_log"], nh)),
            ParamSpec("D", (nh,), kind="vector", init="gain", sources=_src(n["d"], nh)),
            ParamSpec("norm.weight", (self.inner,), kind="vector", init="gain", sources=_src(n["norm"], self.inner)),
            ParamSpec("out_proj.weight", (H, self.inner), sources=_src(n["o"], H)),
        ]

    def product_weights(self) -> tuple[str, ...]:
        return ("in_proj.weight", "out_proj.weight")

    def state_needs(self) -> tuple[StateNeed, ...]:
        return (StateNeed((max(self.taps - 1, 1), self.conv_dim)),
                StateNeed((self.heads, self.state_size, self.head_dim)))

    def check_limits(self, limits) -> None:
        most = ops.ssm_scan_max_state()
        if self.state_size > most:
            raise ValueError(f"a state of {self.state_size} rows a head: the recurrence kernel serves {most}")

    def forward(self, x, ctx, call, sink=None):
        p = self.params
        conv_state, ssm_state = (ctx.states[i] for i in call.state_indices)
        conv_state = conv_state[:, : self.taps - 1]
        batch = dict(positions=ctx.positions, token_req=ctx.token_req, q_start=ctx.q_start,
                     slots=ctx.slots, num_reqs=ctx.num_reqs)
        proj = ctx.buf(f"ssm_proj:{self.proj_dim}", self.proj_dim)
        ops.linear(proj, x, p["in_proj.weight"])
        z = proj[:, : self.inner]
        xbc_raw = proj[:, self.inner: self.inner + self.conv_dim]
        dt_raw = proj[:, self.inner + self.conv_dim:]
        xbc = ctx.buf(f"ssm_xbc:{self.conv_dim}", self.conv_dim, torch.float32)
        ops.causal_conv(xbc, xbc_raw, p["conv.weight"], p["conv.bias"], conv_state, act="silu",
                        single_tokens=ctx.max_query_len == 1, **batch)
        y = ctx.buf(f"ssm_y:{self.inner}", self.inner, torch.float32)
        ops.ssm_scan(y, xbc, dt_raw, p["dt_bias"], p["A_log"], p["D"], ssm_state, heads=self.heads,
                     head_dim=self.head_dim, state_size=self.state_size, groups=self.groups, **batch)
        normed = ctx.buf(f"ssm_normed:{self.inner}", self.inner)
        ops.gated_group_rmsnorm(normed, y, z, p["norm.weight"], self.eps, self.norm_groups)
        out = ctx.buf("mixer_out", self.hidden_size)
        ops.linear(out, normed, p["out_proj.weight"])
        return out


register_mixer("gated_linear_recurrence", GatedLinearRecurrence)
register_mixer("state_space", StateSpaceMixer)
