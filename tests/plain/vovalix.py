"""A plain, slow Vovalix decoder: whole sequences, no cache, no pages, no batching.

One function per mechanism, written from the design's equations in this file's own
notation.  Nothing here imports from the product package; the tests compare the engine
with this file.  Tensors live on the CPU in the dtype of the weights handed in (the tests
use float64).

A model is ``(config, weights)``: the mapping of config.json and a mapping from tensor
name to tensor.  Matrices are ``[out, in]``.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


# ------------------------------------------------------------------ elementwise pieces
def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    """log(1 + e^z), with no threshold above which it turns linear."""
    return torch.logaddexp(z, torch.zeros_like(z))


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x over its root mean square along the last axis, eps inside the root."""
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def offset_rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """The layer norms: the stored weight is the gain minus one."""
    return rms_unit(x, eps) * (1.0 + w)


def unit_vector(x: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """x over its Euclidean length along the last axis, eps inside the root."""
    return x / torch.sqrt(x.pow(2).sum(dim=-1, keepdim=True) + eps)


# ------------------------------------------------------------------------- attention
def distance_slopes(heads: int) -> list[float]:
    """Head h (from 0) loses ``2^(-8 (h + 1) / heads)`` per token of distance."""
    return [2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)]


def chunked_distance_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                               chunk: int | None, eps: float) -> torch.Tensor:
    """``q [T, H, d]``, ``k [T, G, d]``, ``v [T, G, dv]`` of one sequence from position 0.
    Every q and k head is divided by its root mean square; token i scores key j <= i of its own
    chunk (``i // chunk == j // chunk``) as ``q_i . k_j * scale - slope_h (i - j)``; softmax over
    those keys.  Returns ``[T, H, dv]``."""
    T, H, _ = q.shape
    G = k.shape[1]
    q, k = rms_unit(q, eps), rms_unit(k, eps)
    slopes = distance_slopes(H)
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for i in range(T):
        lo = 0 if not chunk else (i // chunk) * chunk
        dist = torch.arange(i - lo, -1, -1, dtype=q.dtype)  # i - j for j = lo .. i
        for h in range(H):
            g = h // (H // G)
            s = (k[lo:i + 1, g] @ q[i, h]) * scale - slopes[h] * dist
            p = torch.softmax(s, dim=0)
            out[i, h] = p @ v[lo:i + 1, g]
    return out


def attention_mixer(x: torch.Tensor, w: dict, p: str, m: dict, eps: float) -> torch.Tensor:
    T = x.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (x @ w[f"{p}.q"].T).view(T, H, d)
    k = (x @ w[f"{p}.k"].T).view(T, G, d)
    v = (x @ w[f"{p}.v"].T).view(T, G, dv)
    chunk = (m.get("mask") or {}).get("size")
    o = chunked_distance_attention(q, k, v, float(m["scale"]), chunk, eps)
    return o.reshape(T, H * dv) @ w[f"{p}.o"].T


# ---------------------------------------------------------------------- recurrences
def gated_linear_recurrence(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor) -> torch.Tensor:
    """One head: ``q, k, decay [T, d]``, ``v [T, dv]``.  ``S_t = decay_t[:, None] * S_(t-1) + k_t
    v_t^T`` from ``S = 0``; ``o_t = S_t^T q_t``."""
    T, d = q.shape
    S = torch.zeros(d, v.shape[1], dtype=q.dtype)
    out = []
    for t in range(T):
        S = decay[t][:, None] * S + torch.outer(k[t], v[t])
        out.append(S.T @ q[t])
    return torch.stack(out)


def delta_recurrence(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, beta: torch.Tensor,
                     g: torch.Tensor) -> torch.Tensor:
    """One head: ``q, k [T, d]``, ``v [T, dv]``, ``beta, g [T]``.  Per token the state shrinks by
    ``g_t``, the value is corrected by what the state already answers for ``k_t``, the
    correction times ``beta_t`` is written at ``k_t``, and the output reads the new state."""
    T, d = q.shape
    S = torch.zeros(d, v.shape[1], dtype=q.dtype)
    out = []
    for t in range(T):
        S = g[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        out.append(S.T @ q[t])
    return torch.stack(out)


def causal_conv(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """``x [T, C]``, ``taps [C, K]``: ``y_t = sum_j taps[:, K-1-j] * x_(t-j)``, zeros before the
    first token."""
    T, _ = x.shape
    K = taps.shape[1]
    y = torch.zeros_like(x)
    for j in range(K):
        y[j:] += x[: T - j] * taps[:, K - 1 - j]
    return y


def head_norm_gate_project(o: torch.Tensor, gate: torch.Tensor, gain: torch.Tensor, w_o: torch.Tensor,
                           eps: float) -> torch.Tensor:
    """``o [T, H, dv]``: every head over its root mean square times ``gain [dv]``, the heads side
    by side times ``silu(gate [T, H dv])``, then the output matrix."""
    T = o.shape[0]
    y = (rms_unit(o, eps) * gain).reshape(T, -1) * silu(gate)
    return y @ w_o.T


def gla_mixer(x: torch.Tensor, w: dict, p: str, m: dict, eps: float) -> torch.Tensor:
    T = x.shape[0]
    H, d, dv, tau = m["heads"], m["dim"], m["vdim"], float(m["tau"])
    q = (x @ w[f"{p}.q"].T).view(T, H, d) * d ** -0.5
    k = (x @ w[f"{p}.k"].T).view(T, H, d)
    v = (x @ w[f"{p}.v"].T).view(T, H, dv)
    z = (x @ w[f"{p}.a1"].T) @ w[f"{p}.a2"].T + w[f"{p}.a2.b"]
    decay = torch.sigmoid(z).pow(1.0 / tau).view(T, H, d)
    o = torch.stack([gated_linear_recurrence(q[:, h], k[:, h], v[:, h], decay[:, h]) for h in range(H)], dim=1)
    return head_norm_gate_project(o, x @ w[f"{p}.g"].T, w[f"{p}.norm"], w[f"{p}.o"], eps)


def delta_mixer(x: torch.Tensor, w: dict, p: str, m: dict, eps: float) -> torch.Tensor:
    T = x.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(x @ w[f"{p}.q"].T, w[f"{p}.q.conv"])).view(T, G, d)
    k = silu(causal_conv(x @ w[f"{p}.k"].T, w[f"{p}.k.conv"])).view(T, G, d)
    v = silu(causal_conv(x @ w[f"{p}.v"].T, w[f"{p}.v.conv"])).view(T, H, dv)
    q = unit_vector(q) * d ** -0.5
    k = unit_vector(k)
    beta = torch.sigmoid(x @ w[f"{p}.b"].T)
    g = torch.exp(-torch.exp(w[f"{p}.A_log"]) * softplus(x @ w[f"{p}.a"].T + w[f"{p}.dt_bias"]))
    o = torch.stack([delta_recurrence(q[:, h // (H // G)], k[:, h // (H // G)], v[:, h], beta[:, h], g[:, h])
                     for h in range(H)], dim=1)
    return head_norm_gate_project(o, x @ w[f"{p}.g"].T, w[f"{p}.norm"], w[f"{p}.o"], eps)


# ---------------------------------------------------------------------- feed-forward
def clamped_glu_expert(x: torch.Tensor, w: dict, p: str, limit: float) -> torch.Tensor:
    g = torch.clamp(x @ w[f"{p}.gate"].T, max=limit)
    u = torch.clamp(x @ w[f"{p}.up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[f"{p}.down"].T


def route(scores: torch.Tensor, top: int, groups: int, keep: int) -> tuple[list[int], torch.Tensor]:
    """``scores [E]`` (a softmax): the ``top`` largest among the experts of the ``keep`` groups
    whose best expert scores highest (``groups`` equal runs of neighbours); their scores over
    their sum.  Ties go to the lower index."""
    E = scores.shape[0]
    per = E // groups
    best = [(float(scores[g * per:(g + 1) * per].max()), -g) for g in range(groups)]
    kept = {-g for _, g in sorted(best, reverse=True)[:keep]}
    allowed = [e for e in range(E) if e // per in kept]
    chosen = sorted(allowed, key=lambda e: (-float(scores[e]), e))[:top]
    weights = scores[chosen]
    return chosen, weights / (weights.sum() + 1e-20)


def route_margin(logits: torch.Tensor, top: int, groups: int, keep: int) -> float:
    """How far the router's choice for ``logits [E]`` is from another one: the smallest gap, in
    units of the logits' spread, between a group that is kept and one that is not, and between an
    expert that is chosen and an allowed one that is not (infinite where there is no other choice)."""
    E = logits.shape[0]
    per = E // groups
    spread = float(logits.std()) if E > 1 else 1.0
    gaps = [float("inf")]
    best = [float(logits[g * per:(g + 1) * per].max()) for g in range(groups)]
    ranked = sorted(range(groups), key=lambda g: (-best[g], g))
    if keep < groups:
        gaps.append(best[ranked[keep - 1]] - best[ranked[keep]])
    allowed = sorted((float(logits[e]) for e in range(E) if e // per in set(ranked[:keep])), reverse=True)
    if top < len(allowed):
        gaps.append(allowed[top - 1] - allowed[top])
    return min(gaps) / (spread + 1e-30)


def moe_feed_forward(x: torch.Tensor, w: dict, p: str, mlp: dict, margins: list | None = None) -> torch.Tensor:
    """``margins``, if given, receives a tensor ``[T]`` of every token's ``route_margin``."""
    r = mlp["router"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    limit = float(mlp["expert"]["limit"])
    logits = x @ w[f"{p}.router"].T
    scores = torch.softmax(logits, dim=-1)
    if margins is not None:
        margins.append(torch.tensor([route_margin(logits[t], r["top"], groups["count"], groups["keep"])
                                     for t in range(x.shape[0])], dtype=torch.float64))
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        chosen, weights = route(scores[t], r["top"], groups["count"], groups["keep"])
        for e, a in zip(chosen, weights):
            out[t] += a * clamped_glu_expert(x[t:t + 1], w, f"{p}.e{e}", limit)[0]
    if mlp.get("shared"):
        out = out + clamped_glu_expert(x, w, f"{p}.shared", float(mlp["shared"]["limit"]))
    return out


# ------------------------------------------------------------------------- the model
MIXERS = {"attention": attention_mixer, "gla": gla_mixer, "delta": delta_mixer}


def vovalix_forward(config: dict, weights: dict, tokens: list[int], dtype=torch.float64,
                    return_layers: bool = False, margins: list | None = None):
    """Logits ``[T, vocab]`` of one sequence from position 0 (and, on request, the stream after
    every layer run, ``[runs, T, width]``).  ``margins``, if given, receives one tensor ``[T]`` per
    routed feed-forward: how clear each token's routing was (``route_margin``)."""
    w = {k: v.to(dtype) for k, v in weights.items()}
    eps = float(config["norm"]["eps"])
    x = w["embed"][torch.tensor(tokens)]
    seen = []
    for i, layer in enumerate(config["layers"]):
        p = f"l{layer['weights_of']}" if layer.get("weights_of") is not None else f"l{i}"
        h = offset_rms_norm(x, w[f"{p}.norm1"], eps)
        y = MIXERS[layer["type"]](h, w, f"{p}.mix", layer["mixer"], eps)
        if layer.get("mlp") is not None:
            y = y + moe_feed_forward(h, w, f"{p}.mlp", layer["mlp"], margins)
        x = x + y
        seen.append(x)
    logits = offset_rms_norm(x, w["final.norm"], eps) @ w["embed"].T * float(config.get("logit_scale", 1.0))
    return (logits, torch.stack(seen)) if return_layers else logits


def load_model_folder(folder: str | Path) -> tuple[dict, dict[str, torch.Tensor]]:
    from safetensors.torch import load_file

    folder = Path(folder)
    config = json.loads((folder / "config.json").read_text())
    weights: dict[str, torch.Tensor] = {}
    for file in sorted(folder.glob("*.safetensors")):
        weights.update(load_file(str(file)))
    return config, weights


def greedy_generate(config: dict, weights: dict, prompt: list[int], n: int, dtype=torch.float64) -> list[int]:
    ids, out = list(prompt), []
    for _ in range(n):
        nxt = int(torch.argmax(vovalix_forward(config, weights, ids, dtype=dtype)[-1]))
        out.append(nxt)
        ids.append(nxt)
    return out
