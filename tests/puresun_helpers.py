"""Tiny Puresun configurations and model folders for the tests.

The configurations differ in every size and option: layer count and order, width (a multiple of 8 or not),
heads (1, 2, 3, 18, 20: more than the 16 that share a KV head in the matrix-core kernels), unrotated / rotated / value sizes,
latent ranks whose cache row is a multiple of 16 or needs padding, windows (4 to 40, none), rotation base,
experts and how many are chosen (all of them, some, one of one), layers without a feed-forward, the
repeated run (at the start, in the middle, once, three times, none), the token-pair table, the logit cap.

Random weights are drawn with a deviation that makes attention scores and router logits of order one, so
that softmax weights are uneven and a wrong key or a lost state changes the logits visibly.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import torch

from reinfer_amd.config import config_from_dict
from reinfer_amd.models import declare_params
from reinfer_amd.weights import random_tensors
from reinfer_amd.weights.safetensors_io import write_safetensors


def _mixer(heads, dim, rot_dim, vdim, rank, window, base=10000.0, dims=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank,
         "scale": 1.0 / math.sqrt(dim + rot_dim), "rot": {"base": base, "dims": rot_dim if dims is None else dims}}
    if window:
        m["mask"] = {"size": window}
    return m


def _moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def _layer(mixer, mlp):
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


# three layers, the last two run three times; two window sizes (two cache groups); a layer with no feed-forward;
# cache rows of 48 (no padding) and 40 -> 48 (padding); rotation on part of the rotated entries in layer 1
PS_A = {
    "architecture": "Puresun", "vocab": 300, "width": 48, "norm": {"eps": 1e-6}, "logit_softcap": 20.0,
    "embedding": {"bigram": {"buckets": 97, "mul_prev": 13, "mul_cur": 5}},
    "layers": [
        _layer(_mixer(3, 16, 8, 24, 40, 21), _moe(5, 2, 24)),
        _layer(_mixer(2, 8, 16, 16, 24, 9, base=500.0, dims=8), None),
        _layer(_mixer(3, 16, 8, 8, 40, 21), _moe(3, 3, 40)),
    ],
    "loop": {"start": 1, "stop": 3, "times": 3},
}
# no pair table, no repeated run, no cap; one head; every expert chosen; one expert of one; a window of 4
PS_B = {
    "architecture": "Puresun", "vocab": 257, "width": 64, "norm": {"eps": 1e-5},
    "layers": [
        _layer(_mixer(1, 32, 16, 32, 64, 4), _moe(4, 4, 16)),
        _layer(_mixer(18, 16, 16, 8, 48, 40, base=1000000.0), _moe(1, 1, 72)),
    ],
}
# a width that is no multiple of 8, 20 heads, a cache row of 106 -> 112, no window on the second layer,
# the first layer repeated twice, the run of one pass in between is the whole loop
PS_C = {
    "architecture": "Puresun", "vocab": 131, "width": 36, "norm": {"eps": 3e-6}, "logit_softcap": 7.5,
    "embedding": {"bigram": {"buckets": 31, "mul_prev": 3, "mul_cur": 11}},
    "layers": [
        _layer(_mixer(20, 8, 6, 4, 100, 13, base=77.0), _moe(7, 3, 10)),
        _layer(_mixer(2, 24, 8, 20, 16, 0), _moe(2, 1, 20)),
    ],
    "loop": {"start": 0, "stop": 1, "times": 2},
}
# for bfloat16: as A, but every feed-forward uses all its experts, so that no comparison rests on which of
# two nearly equal router logits is the larger after rounding
PS_A16 = json.loads(json.dumps(PS_A))
PS_A16["layers"][0]["mlp"] = _moe(4, 4, 24)

# a latent wider than the matrix-core attention kernels' largest head (288 > 256): the plain kernel in both dtypes
PS_D = {
    "architecture": "Puresun", "vocab": 90, "width": 32, "norm": {"eps": 1e-6},
    "embedding": {"bigram": {"buckets": 10, "mul_prev": 1, "mul_cur": 1}},
    "layers": [_layer(_mixer(2, 8, 8, 8, 280, 12), _moe(2, 2, 8))],
    "loop": {"start": 0, "stop": 1, "times": 1},
}

CONFIGS = {"A": (PS_A, 11), "B": (PS_B, 12), "C": (PS_C, 13), "A16": (PS_A16, 14), "D": (PS_D, 15)}

# deviation of the random matrices by the last part of their name (norm weights are uniform on [0.8, 1.2))
STD = {"embed": 1.0, "bigram": 0.5, "loop.step": 0.5, "router": 0.6, "head": 0.3, "default": 0.15}


def draw_weights(raw: dict, seed: int, dtype: torch.dtype = torch.float32, scales: Optional[Dict[str, float]] = None):
    """name -> tensor of the random model of ``raw`` and ``seed``; ``scales`` multiplies named tensors."""
    cfg = config_from_dict(raw)
    decls = declare_params(cfg.to_spec())
    out = {}
    for d in decls:
        if d.optional:
            continue
        key = d.name if d.name in STD else d.name.rsplit(".", 1)[-1]
        std = STD.get(key, STD["default"])
        out.update(random_tensors([d], seed, torch.float32, std=std))
    for name, f in (scales or {}).items():
        out[name] = out[name] * f
    return {n: t.to(dtype) for n, t in out.items()}


def make_folder(tmp_path, which: str, dtype: str = "bfloat16", scales: Optional[Dict[str, float]] = None,
                tag: str = "") -> str:
    raw, seed = CONFIGS[which]
    out = os.path.join(str(tmp_path), f"puresun_{which}_{dtype}{tag}")
    if not os.path.isdir(out):
        os.makedirs(out)
        tdtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
        with open(os.path.join(out, "config.json"), "w", encoding="utf-8") as f:
            json.dump(raw, f, indent=1)
        write_safetensors(os.path.join(out, "model.safetensors"), draw_weights(raw, seed, tdtype, scales),
                          metadata={"format": "pt"})
    return out


def read_folder(path: str, dtype=torch.float64):
    """(raw config dict, name -> CPU tensor in ``dtype``) for the plain implementation."""
    from reinfer_amd.weights import SafetensorsFile
    with open(os.path.join(path, "config.json")) as f:
        raw = json.load(f)
    with SafetensorsFile(os.path.join(path, "model.safetensors")) as sf:
        weights = {n: sf.tensor(n).to(dtype) for n in sf.names()}
    return raw, weights
