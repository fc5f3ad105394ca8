"""Configurations, model folders and batch helpers for the Vovalix tests.

The configurations differ from each other in every size and option: layer order, widths, head
counts and grouping, key and value sizes (different and equal), chunk sizes (down to one
position, and none), convolution taps, expert counts, groups and choices, layers without a
feed-forward, feed-forwards without a shared expert, layers that run another layer's tensors,
and values that are 1 or equal where another model's differ.
"""

from __future__ import annotations

import json
from pathlib import Path

import torch


def _attn(heads, kv, dim, vdim, scale, chunk):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if chunk:
        m["mask"] = {"size": chunk}
    return m


def _gla(heads, dim, vdim, tau, rank):
    return {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "rank": rank}


def _delta(heads, kv, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv}


def _moe(experts, top, ff, limit, groups=None, shared=None):
    router = {"experts": experts, "top": top}
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    m = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": router}
    if shared:
        m["shared"] = {"ff": shared[0], "limit": shared[1]}
    return m


_MOE_A = _moe(6, 2, 40, 1.0, groups=(3, 2), shared=(56, 2.0))
_GLA_A = _gla(3, 24, 40, 8.0, 12)

# keys of 32 and values of 16 under grouped heads, chunks of 24 positions (pages of 8), a gated
# linear layer that runs twice with the same tensors, a last layer without a feed-forward
CONFIG_A = {
    "architecture": "Vovalix", "vocab": 211, "width": 96, "norm": {"eps": 1e-5}, "logit_scale": 1.5,
    "layers": [
        {"type": "attention", "mixer": _attn(4, 2, 32, 16, 0.2, 24), "mlp": _MOE_A},
        {"type": "gla", "mixer": _GLA_A, "mlp": _MOE_A},
        {"type": "delta", "mixer": _delta(4, 2, 24, 20, 3), "mlp": _moe(5, 3, 24, 0.7, shared=(16, 0.5))},
        {"type": "gla", "mixer": _GLA_A, "mlp": _MOE_A, "weights_of": 1},
        {"type": "attention", "mixer": _attn(6, 6, 16, 16, 0.25, 10), "mlp": None},
    ],
}

# keys and values of 64 with four query heads a kv head, pages of 16: the shapes the matrix-core
# attention kernels serve in bfloat16; chunks of 48 (not a multiple of the kernels' tiles); experts
# without groups and without a shared expert; a delta layer whose every head has its own keys
CONFIG_B = {
    "architecture": "Vovalix", "vocab": 320, "width": 128, "norm": {"eps": 1e-6}, "logit_scale": 0.5,
    "layers": [
        {"type": "delta", "mixer": _delta(2, 2, 64, 64, 4), "mlp": _moe(8, 3, 64, 2.0)},
        {"type": "attention", "mixer": _attn(8, 2, 64, 64, 0.125, 48), "mlp": _moe(8, 3, 64, 2.0)},
        {"type": "gla", "mixer": _gla(2, 64, 64, 12.0, 24), "mlp": _moe(4, 1, 128, 3.0, groups=(2, 1), shared=(64, 1.0))},
        {"type": "attention", "mixer": _attn(8, 2, 64, 64, 0.125, 48), "mlp": _moe(8, 3, 64, 2.0), "weights_of": 1},
    ],
}

# ones and equal values: one head, one kv head, a chunk of one position (a token sees itself
# only) beside a layer that sees everything, values twice as wide as keys, a convolution of one
# tap, a decay product of rank 1, two experts of which both are chosen, an odd vocabulary
CONFIG_C = {
    "architecture": "Vovalix", "vocab": 97, "width": 40, "norm": {"eps": 1e-4},
    "layers": [
        {"type": "gla", "mixer": _gla(1, 8, 5, 1.0, 1), "mlp": _moe(2, 2, 8, 0.3, groups=(2, 2))},
        {"type": "attention", "mixer": _attn(1, 1, 16, 32, 1.0, 1), "mlp": None},
        {"type": "delta", "mixer": _delta(1, 1, 8, 1, 1), "mlp": _moe(3, 1, 16, 5.0, groups=(3, 1))},
        {"type": "attention", "mixer": _attn(2, 1, 16, 16, 0.5, 0), "mlp": _moe(2, 1, 24, 1.0, shared=(8, 1.0))},
        {"type": "delta", "mixer": _delta(3, 1, 8, 1, 1), "mlp": None},
    ],
}

# wide states: 200 key channels a head (many rows a thread), 80 value channels a head (more than
# one tile), sixteen experts in four groups of which one is kept, five taps
CONFIG_D = {
    "architecture": "Vovalix", "vocab": 256, "width": 64, "norm": {"eps": 1e-6}, "logit_scale": 3.0,
    "layers": [
        {"type": "gla", "mixer": _gla(2, 200, 80, 4.0, 8), "mlp": _moe(16, 4, 32, 1.0, groups=(4, 1), shared=(32, 1.0))},
        {"type": "delta", "mixer": _delta(2, 1, 130, 72, 5), "mlp": _moe(16, 4, 32, 1.0, groups=(4, 2))},
        {"type": "attention", "mixer": _attn(3, 1, 48, 72, 0.15, 100), "mlp": None},
    ],
}

CONFIGS = {"A": (CONFIG_A, 8), "B": (CONFIG_B, 16), "C": (CONFIG_C, 4), "D": (CONFIG_D, 16)}


def random_config(rng) -> dict:
    """A configuration drawn from ``rng`` (a ``random.Random``): three to eight layers of any kind in any
    order, some borrowing an earlier layer's tensors, some without a feed-forward; widths, head counts
    and grouping, key and value sizes, chunks, taps, ranks, experts, groups and choices all drawn anew."""
    width = rng.choice([64, 96, 128, 192, 256, 320, 100])
    def moe():
        groups = rng.choice([1, 2, 3, 4])
        per = rng.choice([1, 2, 3, 4])
        E = groups * per
        keep = rng.randint(1, groups)
        top = rng.randint(1, min(4, keep * per))
        m = {"kind": "moe", "expert": {"ff": rng.choice([24, 32, 48, 64, 96, 40]), "limit": rng.choice([0.5, 1.0, 2.5])},
             "router": {"experts": E, "top": top}}
        if groups > 1 or rng.random() < 0.5:  # a single group may also go unsaid
            m["router"]["groups"] = {"count": groups, "keep": keep}
        if rng.random() < 0.6: m["shared"] = {"ff": rng.choice([16, 64, 128, 72]), "limit": rng.choice([0.7, 1.5])}
        return m
    def attn():
        kv = rng.choice([1, 2, 3, 4]); g = rng.choice([1, 2, 4])
        dim = rng.choice([16, 32, 48, 64, 64, 128]); vdim = rng.choice([dim, dim, 2 * dim if dim <= 64 else dim, 24, 80])
        m = {"heads": kv * g, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": rng.choice([0.125, 0.2, 0.09])}
        if rng.random() < 0.85: m["mask"] = {"size": rng.choice([7, 16, 33, 64, 100, 128, 50])}
        return m
    def gla():
        return {"heads": rng.choice([1, 2, 3, 6]), "dim": rng.choice([8, 16, 32, 48, 64, 20]), "vdim": rng.choice([16, 64, 32, 40, 128]),
                "tau": rng.choice([4.0, 16.0, 7.5]), "rank": rng.choice([4, 8, 16, 5])}
    def delta():
        kv = rng.choice([1, 2, 3]); g = rng.choice([1, 2])
        return {"heads": kv * g, "kv_heads": kv, "dim": rng.choice([16, 32, 64, 128, 24]), "vdim": rng.choice([16, 32, 64, 128, 40]),
                "conv": rng.choice([1, 2, 3, 4])}
    kinds = {"attention": attn, "gla": gla, "delta": delta}
    layers = []
    for i in range(rng.randint(3, 8)):
        own = [j for j, l in enumerate(layers) if "weights_of" not in l]
        if own and rng.random() < 0.3:
            j = rng.choice(own)
            l = dict(layers[j]); l["weights_of"] = j
            layers.append(l); continue
        t = rng.choice(list(kinds))
        layers.append({"type": t, "mixer": kinds[t](), "mlp": moe() if rng.random() < 0.85 else None})
    return {"architecture": "Vovalix", "vocab": rng.choice([97, 256, 512, 1000]), "width": width,
            "norm": {"eps": rng.choice([1e-6, 1e-5])}, "logit_scale": rng.choice([1.0, 2.0, 0.5]), "layers": layers}


def make_model_dir(folder: Path, config: dict, seed: int) -> Path:
    """A model folder from the product's random-weights mode, with the small tensors redrawn so
    that each one matters: biases and decay parameters get values that spread the decays between
    fast and slow, the routers get weights that send tokens to every expert, the norms' stored
    weights lie around zero, and the matrices are livelier than N(0, 0.02)."""
    from safetensors.torch import load_file, save_file

    from kvcore_amd.weights.loader import write_random_model

    write_random_model(folder, config, seed)
    path = folder / "model.safetensors"
    tensors = load_file(str(path))
    gen = torch.Generator().manual_seed(seed + 1)

    def noise(t, std, mean=0.0):
        return (torch.randn(t.shape, generator=gen) * std + mean).to(torch.bfloat16).to(t.dtype)

    for name, t in list(tensors.items()):
        leaf = name.split(".")[-1]
        if name.endswith("a2.b"):
            tensors[name] = noise(t, 1.0, 2.0)
        elif leaf == "dt_bias":
            tensors[name] = noise(t, 0.5)
        elif leaf == "conv":
            tensors[name] = noise(t, 0.4)
        elif leaf == "A_log":
            tensors[name] = noise(t, 0.7, -0.5)
        elif leaf == "router":
            tensors[name] = noise(t, 0.3)
        elif leaf == "norm1" or name == "final.norm":
            tensors[name] = noise(t, 0.2)
        elif leaf == "norm":
            tensors[name] = noise(t, 0.2, 1.0)
        elif name == "embed":
            tensors[name] = noise(t, 1.0)
        elif t.dim() == 2:
            tensors[name] = noise(t, 0.08)
    save_file(tensors, str(path))
    return folder


def batch_tensors(reqs, device="cuda"):
    """``reqs``: (slot, first position, number of tokens) per request, or None for a padded
    request of one padding token -> positions, token_req, q_start, slots (int32 on the device)
    and the number of tokens."""
    positions, token_req, q_start, slots = [], [], [0], []
    for r, item in enumerate(reqs):
        if item is None:
            positions.append(0)
            token_req.append(-1)
            slots.append(0)
        else:
            slot, start, n = item
            positions += list(range(start, start + n))
            token_req += [r] * n
            slots.append(slot)
        q_start.append(len(positions))

    def dev(v):
        return torch.tensor(v, dtype=torch.int32, device=device)

    return dict(positions=dev(positions), token_req=dev(token_req), q_start=dev(q_start), slots=dev(slots),
                num_reqs=len(reqs)), len(positions)
