"""A plain, slow Dirulorn decoder: whole sequences, no cache, no pages, no batching.

One function per mechanism, written from the design's equations in this file's own
notation.  Nothing here imports from the product package; the tests compare the engine
with this file.  Tensors live on the CPU in the dtype of the weights handed in (the tests
use float64).

A model is ``(config, weights)``: the mapping of config.json and a mapping from tensor
name to tensor.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


# ------------------------------------------------------------------ elementwise pieces
def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    """log(1 + e^z), with no threshold above which it turns linear."""
    return torch.logaddexp(z, torch.zeros_like(z))


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x over its root mean square along the last axis, eps inside the root."""
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def layer_norm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    mu = x.mean(dim=-1, keepdim=True)
    var = (x - mu).pow(2).mean(dim=-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


# -------------------------------------------------------------------------- rotation
def rotary_frequencies(dims: int, base: float, scaling: dict | None) -> list[float]:
    """f_i = base^(-2i/dims); with ``scaling`` (factor, low, high, original) the long
    wavelengths are slowed by ``factor``, the short ones kept, and those between blended."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high = float(scaling["factor"]), float(scaling["low"]), float(scaling["high"])
            orig = float(scaling["original"])
            lam = 2.0 * math.pi / f
            if lam < orig / high:
                pass
            elif lam > orig / low:
                f = f / factor
            else:
                s = (orig / lam - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return out


def rotate_interleaved(x: torch.Tensor, freqs: list[float], first_pos: int = 0) -> torch.Tensor:
    """``x [T, heads, d]``: pair (2i, 2i+1) of the first ``2 len(freqs)`` elements of each head
    is turned by the angle ``position * f_i``; the rest passes."""
    T = x.shape[0]
    out = x.clone()
    pos = torch.arange(first_pos, first_pos + T, dtype=x.dtype)
    for i, f in enumerate(freqs):
        ang = pos * f
        c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


# ------------------------------------------------------------------------- attention
def softmax_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float) -> torch.Tensor:
    """``q [T, H, d]``, ``k [T, G, d]``, ``v [T, G, dv]`` -> ``[T, H, dv]``; causal; query head
    h reads key/value head ``h // (H / G)``."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.empty(T, H, v.shape[2], dtype=q.dtype)
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool))
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~mask, float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def attention_branch(h: torch.Tensor, w: dict, p: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + ".q"].T).view(T, H, d)
    k = (h @ w[p + ".k"].T).view(T, G, d)
    v = (h @ w[p + ".v"].T).view(T, G, dv)
    q = rms_unit(q, eps) * w[p + ".q.norm"]
    k = rms_unit(k, eps) * w[p + ".k.norm"]
    rot = m.get("rot")
    if rot:
        freqs = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q, k = rotate_interleaved(q, freqs), rotate_interleaved(k, freqs)
    o = softmax_attention(q, k, v, float(m["scale"]))
    return o.reshape(T, H * dv) @ w[p + ".o"].T


# ------------------------------------------------------------------ short convolution
def causal_conv(x: torch.Tensor, taps: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """``x [T, C]``, ``taps [C, K]``: out[t] = bias + sum_j taps[:, K-1-j] * x[t-j], zeros
    before the start."""
    T, C = x.shape
    K = taps.shape[1]
    out = bias.expand(T, C).clone()
    for j in range(K):
        if j < T:
            out[j:] += taps[:, K - 1 - j] * x[: T - j]
    return out


# ------------------------------------------------------- gated linear recurrent unit
def recurrent_branch(h: torch.Tensor, w: dict, p: str, m: dict) -> torch.Tensor:
    T = h.shape[0]
    width, nb = m["width"], m["blocks"]
    y = gelu_tanh(h @ w[p + ".y"].T + w[p + ".y.b"])
    u = causal_conv(h @ w[p + ".x"].T + w[p + ".x.b"], w[p + ".conv"], w[p + ".conv.b"])
    ub = u.view(T, nb, width // nb)
    r = torch.sigmoid(torch.einsum("boi,tbi->tbo", w[p + ".ra"], ub) + w[p + ".ra.b"]).reshape(T, width)
    i = torch.sigmoid(torch.einsum("boi,tbi->tbo", w[p + ".ri"], ub) + w[p + ".ri.b"]).reshape(T, width)
    log_a = -8.0 * r * softplus(w[p + ".lam"])
    a = torch.exp(log_a)
    drive = torch.sqrt(1.0 - a * a) * i * u
    S = torch.zeros(width, dtype=h.dtype)
    states = torch.empty(T, width, dtype=h.dtype)
    for t in range(T):
        S = a[t] * S + drive[t]
        states[t] = S
    return (states * y) @ w[p + ".o"].T


def parallel_mixer(h: torch.Tensor, w: dict, p: str, m: dict, eps: float) -> torch.Tensor:
    left = attention_branch(h, w, p + ".left", m["left"], eps)
    right = recurrent_branch(h, w, p + ".right", m["right"])
    return 0.5 * (rms_unit(left, eps) * w[p + ".left.out"] + rms_unit(right, eps) * w[p + ".right.out"])


# ------------------------------------------------------------------ state-space mixer
def mamba2_mixer(h: torch.Tensor, w: dict, p: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    nh, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = nh * P
    proj = h @ w[p + ".in"].T
    z = proj[:, :inner]
    xbc = proj[:, inner: 2 * inner + 2 * G * N]
    dt = proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[p + ".conv"], w[p + ".conv.b"]))
    x = xbc[:, :inner].view(T, nh, P)
    B = xbc[:, inner: inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + w[p + ".dt_bias"])
    decay = torch.exp(-torch.exp(w[p + ".A_log"]) * dt)  # [T, nh]
    y = torch.empty(T, nh, P, dtype=h.dtype)
    for hd in range(nh):
        g = hd // (nh // G)
        S = torch.zeros(N, P, dtype=h.dtype)
        for t in range(T):
            S = decay[t, hd] * S + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S.T @ C[t, g] + w[p + ".D"][hd] * x[t, hd]
    y = y.reshape(T, inner) * silu(z)
    ng = m["norm_groups"]
    y = rms_unit(y.view(T, ng, inner // ng), eps).reshape(T, inner) * w[p + ".norm"]
    return y @ w[p + ".o"].T


# ------------------------------------------------------------------------ feed-forward
def dense_ff(h: torch.Tensor, w: dict, p: str) -> torch.Tensor:
    return (silu(h @ w[p + ".gate"].T) * (h @ w[p + ".up"].T)) @ w[p + ".down"].T


# ----------------------------------------------------------------------------- model
def run_layer(x: torch.Tensor, cfg: dict, w: dict, i: int) -> torch.Tensor:
    layer = cfg["layers"][i]
    eps = float(cfg["norm"]["eps"])
    p = f"l{i}"
    h = layer_norm(x, w[p + ".norm1"], w[p + ".norm1.b"], eps)
    if layer["type"] == "parallel":
        x = x + parallel_mixer(h, w, p + ".mix", layer["mixer"], eps)
    elif layer["type"] == "mamba2":
        x = x + mamba2_mixer(h, w, p + ".mix", layer["mixer"], eps)
    else:
        raise ValueError(f"unknown layer type {layer['type']!r}")
    if layer.get("mlp"):
        if layer["mlp"]["kind"] != "dense":
            raise ValueError(f"unknown feed-forward kind {layer['mlp']['kind']!r}")
        x = x + dense_ff(layer_norm(x, w[p + ".norm2"], w[p + ".norm2.b"], eps), w, p + ".mlp")
    return x


def layer_runs(cfg: dict) -> list[tuple[int, int | None]]:
    """The order in which layers run: (layer, pass number if this run opens a pass)."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    runs = [(i, None) for i in range(start)]
    for t in range(times):
        for i in range(start, stop):
            runs.append((i, t if i == start else None))
    runs += [(i, None) for i in range(stop, n)]
    return runs


def forward(cfg: dict, w: dict, tokens: list[int], keep_layers: bool = False):
    """Logits ``[T, vocab]`` for one whole sequence (and the stream after every layer run)."""
    eps = float(cfg["norm"]["eps"])
    x0 = w["embed"][torch.tensor(tokens)]
    x = x0
    kept = []
    for i, opens in layer_runs(cfg):
        if opens is not None:
            x = torch.cat([x, x0], dim=-1) @ w["loop.in"].T + w["loop.step"][opens]
        x = run_layer(x, cfg, w, i)
        kept.append(x)
    logits = layer_norm(x, w["final.norm"], w["final.norm.b"], eps) @ w["head"].T
    return (logits, torch.stack(kept)) if keep_layers else logits


def load_model_folder(folder: str | Path, dtype=torch.float64):
    from safetensors import safe_open

    folder = Path(folder)
    cfg = json.loads((folder / "config.json").read_text())
    w = {}
    with safe_open(str(folder / "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            w[name] = t.to(dtype) if t.dtype.is_floating_point else t
    return cfg, w
