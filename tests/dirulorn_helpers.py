"""Configurations, model folders and batch helpers for the Dirulorn tests.

The configurations differ from each other in every size and option: layer order, widths, head
counts and grouping, key and value sizes (different and equal), rotation (partial, whole,
with and without rescaling, none), convolution taps, state and block counts, a layer without a
feed-forward, a loop over some layers or none, and values that are 1 or equal where another
model's differ.
"""

from __future__ import annotations

import json
from pathlib import Path

import torch


def _ssm(heads, vdim, state, groups, conv, norm_groups):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
            "norm_groups": norm_groups}


def _par(heads, kv, dim, vdim, scale, rot, width, blocks, conv):
    left = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if rot is not None:
        left["rot"] = rot
    return {"left": left, "right": {"width": width, "blocks": blocks, "conv": conv}}


# keys of 32 and values of 16 under grouped heads, a partial rescaled rotation, a loop over the
# middle layers, a layer without a feed-forward
CONFIG_P = {
    "architecture": "Dirulorn", "vocab": 211, "width": 96, "norm": {"eps": 1e-5},
    "layers": [
        {"type": "parallel", "mlp": {"kind": "dense", "ff": 160},
         "mixer": _par(4, 2, 32, 16, 0.2, {"dims": 8, "base": 5000.0, "scaling":
                       {"factor": 4.0, "low": 1.0, "high": 2.0, "original": 24}}, 72, 3, 3)},
        {"type": "mamba2", "mlp": None, "mixer": _ssm(6, 20, 24, 3, 3, 3)},
        {"type": "parallel", "mlp": {"kind": "dense", "ff": 112},
         "mixer": _par(6, 3, 24, 40, 0.31, {"dims": 24, "base": 300.0}, 64, 4, 5)},
        {"type": "mamba2", "mlp": {"kind": "dense", "ff": 200}, "mixer": _ssm(4, 16, 40, 1, 2, 1)},
    ],
    "loop": {"start": 1, "stop": 3, "times": 3},
}

# keys and values of one size (64) with four query heads a kv head, and values of three times
# the keys' size (kept as three planes of 64): in bfloat16 with pages of 16 the matrix-core
# attention kernels serve both; no loop
CONFIG_Q = {
    "architecture": "Dirulorn", "vocab": 320, "width": 128, "norm": {"eps": 1e-6},
    "layers": [
        {"type": "mamba2", "mlp": {"kind": "dense", "ff": 192}, "mixer": _ssm(4, 64, 128, 2, 4, 2)},
        {"type": "parallel", "mlp": {"kind": "dense", "ff": 192},
         "mixer": _par(8, 2, 64, 64, 0.125, {"dims": 32, "base": 10000.0, "scaling":
                       {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}}, 128, 2, 4)},
        {"type": "parallel", "mlp": {"kind": "dense", "ff": 256},
         "mixer": _par(4, 2, 64, 192, 0.11, None, 96, 1, 2)},  # values three times as wide as keys
    ],
}

# ones and equal values: one head, one group, one block, one kv head, a convolution of one tap
# and of two, a state of 3 rows, value channels of 1 and 5, an odd vocabulary; the whole model
# is the loop
CONFIG_R = {
    "architecture": "Dirulorn", "vocab": 97, "width": 40, "norm": {"eps": 1e-4},
    "layers": [
        {"type": "mamba2", "mlp": {"kind": "dense", "ff": 40}, "mixer": _ssm(1, 5, 3, 1, 1, 1)},
        {"type": "parallel", "mlp": None,
         "mixer": _par(1, 1, 16, 32, 1.0, {"dims": 2, "base": 2.0}, 40, 1, 1)},
        {"type": "mamba2", "mlp": None, "mixer": _ssm(7, 1, 9, 7, 2, 7)},
    ],
    "loop": {"start": 0, "stop": 3, "times": 2},
}

# a wide state (200 rows a head) and 80 value channels a head (more than one tile), keys of 48
CONFIG_S = {
    "architecture": "Dirulorn", "vocab": 256, "width": 64, "norm": {"eps": 1e-6},
    "layers": [
        {"type": "mamba2", "mlp": {"kind": "dense", "ff": 96}, "mixer": _ssm(2, 80, 200, 1, 4, 4)},
        {"type": "parallel", "mlp": {"kind": "dense", "ff": 96},
         "mixer": _par(3, 1, 48, 72, 0.15, {"dims": 48, "base": 100.0}, 160, 2, 4)},
    ],
    "loop": {"start": 1, "stop": 2, "times": 2},
}

# state-space layers only: a model that keeps no paged cache at all, only states
CONFIG_M = {
    "architecture": "Dirulorn", "vocab": 150, "width": 48, "norm": {"eps": 1e-5},
    "layers": [
        {"type": "mamba2", "mlp": {"kind": "dense", "ff": 64}, "mixer": _ssm(2, 16, 8, 1, 3, 1)},
        {"type": "mamba2", "mlp": {"kind": "dense", "ff": 80}, "mixer": _ssm(4, 24, 32, 2, 4, 2)},
    ],
}

CONFIGS = {"P": (CONFIG_P, 8), "Q": (CONFIG_Q, 16), "R": (CONFIG_R, 4), "S": (CONFIG_S, 16), "M": (CONFIG_M, 16)}


def make_model_dir(folder: Path, config: dict, seed: int) -> Path:
    """A model folder from the product's random-weights mode, with the small tensors redrawn so
    that each one matters: biases and steps (which that mode leaves at zero or tiny) get noise,
    and the decay parameters get values that spread the decays between fast and slow."""
    from safetensors.torch import load_file, save_file

    from kvcore_amd.weights.loader import write_random_model

    write_random_model(folder, config, seed)
    path = folder / "model.safetensors"
    tensors = load_file(str(path))
    gen = torch.Generator().manual_seed(seed + 1)

    def noise(t, std, mean=0.0):
        return (torch.randn(t.shape, generator=gen) * std + mean).to(torch.bfloat16).to(t.dtype)

    for name, t in list(tensors.items()):
        leaf = name.split(".mix.")[-1] if ".mix." in name else name
        if name.endswith(".b") or leaf in ("dt_bias",) or name == "loop.step":
            tensors[name] = noise(t, 0.3)
        elif leaf.endswith("conv"):
            tensors[name] = noise(t, 0.4)
        elif leaf == "A_log":
            tensors[name] = noise(t, 0.7, -0.5)
        elif leaf.endswith("lam"):
            tensors[name] = noise(t, 1.0, -2.0)
        elif leaf in ("left.ra", "left.ri", "right.ra", "right.ri"):
            tensors[name] = noise(t, 0.3)
        elif leaf == "D":
            tensors[name] = noise(t, 0.5, 1.0)
        elif t.dim() == 2 and t.dtype == torch.bfloat16:
            tensors[name] = noise(t, 0.08)  # livelier products than N(0, 0.02)
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


def read_config(folder: Path) -> dict:
    return json.loads((Path(folder) / "config.json").read_text())
