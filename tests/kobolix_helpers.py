"""Tiny Kobolix configurations and model folders for the tests.

The configurations differ in every size and option: layer order (a side-by-side layer first or last, matrix-memory
layers alone), width (a multiple of 8 or not), the residual factor and the embedding's scale (also 1 and absent),
attention heads in groups of 1 and 2 with key sizes that are no multiple of 16 and value sizes above and below them,
rotation on all or on part of a head, delta-rule heads on one shared or on their own key heads, key sizes on either
side of the scan kernels' switch from 8 to 32 lanes a column, filters of 1, 3 and 4 taps, experts in groups
(2 of 4 kept), in one group, all chosen, with and without a shared expert, layers with no feed-forward.

Random weights are drawn so that attention scores, gates and router logits are of order one: softmax weights are
uneven, the forget gates sit between 0.5 and 1, and a wrong key or a lost state changes the logits visibly.
"""
from __future__ import annotations

import json
import os
from typing import Dict, Optional

import torch

from reinfer_amd.config import config_from_dict
from reinfer_amd.models import declare_params
from reinfer_amd.weights import random_tensors
from reinfer_amd.weights.safetensors_io import write_safetensors


def _attn(heads, kv, dim, vdim, dims, base=10000.0, scale=None):
    return {"dim": dim, "heads": heads, "kv_heads": kv, "rot": {"base": base, "dims": dims},
            "scale": dim ** -0.5 if scale is None else scale, "vdim": vdim}


def _delta(heads, kv, dim, vdim, conv):
    return {"conv": conv, "dim": dim, "heads": heads, "kv_heads": kv, "vdim": vdim}


def _memory(heads, dim, vdim, cap):
    return {"dim": dim, "gate_cap": cap, "heads": heads, "vdim": vdim}


def _moe(experts, top, ff, groups=None, scale=1.0, shared=0):
    router = {"experts": experts, "scale": scale, "top": top}
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    out = {"expert": {"ff": ff}, "kind": "moe", "router": router}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def _dense(ff):
    return {"ff": ff, "kind": "dense"}


KB_A = {
    "architecture": "Kobolix", "vocab": 300, "width": 64, "norm": {"eps": 1e-5}, "residual_mult": 0.5,
    "embedding": {"scale": 4.0},
    "layers": [
        {"type": "parallel", "mixer": {"left": _attn(4, 2, 24, 16, 12), "right": _delta(4, 1, 20, 12, 3)},
         "mlp": _moe(8, 2, 24, groups=(4, 2), scale=1.5, shared=40)},
        {"type": "mlstm", "mixer": _memory(3, 20, 28, 10.0), "mlp": _dense(96)},
        {"type": "mlstm", "mixer": _memory(1, 40, 8, 15.0), "mlp": None},
        {"type": "parallel", "mixer": {"left": _attn(2, 2, 16, 48, 16, base=500.0, scale=0.3),
                                       "right": _delta(2, 2, 136, 8, 1)},
         "mlp": _moe(6, 6, 16)},
    ],
}
# matrix-memory layers alone: no keys, so no block pool; a width that is no multiple of 8; every factor 1 or absent
KB_B = {
    "architecture": "Kobolix", "vocab": 131, "width": 36, "norm": {"eps": 3e-6}, "residual_mult": 1.0,
    "layers": [
        {"type": "mlstm", "mixer": _memory(2, 12, 20, 8.0), "mlp": _dense(40)},
        {"type": "mlstm", "mixer": _memory(4, 9, 5, 20.0), "mlp": None},
    ],
}
# for bfloat16: no comparison rests on which of two nearly equal scores is the larger after rounding (every
# expert of the one group is chosen); a filter of 4 taps; one attention head a KV head and eight on one
KB_C = {
    "architecture": "Kobolix", "vocab": 257, "width": 96, "norm": {"eps": 1e-6}, "residual_mult": 0.7,
    "embedding": {"scale": 2.0},
    "layers": [
        {"type": "mlstm", "mixer": _memory(2, 32, 48, 11.0), "mlp": _moe(4, 4, 32, scale=0.5, shared=16)},
        {"type": "parallel", "mixer": {"left": _attn(8, 1, 32, 32, 8, base=100000.0), "right": _delta(6, 3, 16, 24, 4)},
         "mlp": _dense(128)},
        {"type": "parallel", "mixer": {"left": _attn(3, 3, 40, 24, 40), "right": _delta(1, 1, 64, 40, 2)},
         "mlp": None},
    ],
}
# whatever may be absent is absent: no rotation, no cap on the gates, no score scale given (1 / sqrt(size)), no groups,
# no router scale, no shared expert, no embedding scale, no residual factor; one expert of one; a side-by-side layer first
KB_D = {
    "architecture": "Kobolix", "vocab": 90, "width": 40, "norm": {"eps": 1e-6},
    "layers": [
        {"type": "parallel", "mixer": {"left": {"dim": 16, "heads": 5, "kv_heads": 5, "vdim": 8},
                                       "right": _delta(3, 1, 8, 16, 2)},
         "mlp": {"expert": {"ff": 24}, "kind": "moe", "router": {"experts": 1, "top": 1}}},
        {"type": "mlstm", "mixer": {"dim": 8, "heads": 5, "vdim": 8}, "mlp": _dense(56)},
    ],
}
CONFIGS = {"A": (KB_A, 21), "B": (KB_B, 22), "C": (KB_C, 23), "D": (KB_D, 24)}

# deviation of the random matrices by the last part of their name
STD = {"embed": 0.5, "router": 0.5, "conv": 0.6, "i": 0.3, "f": 0.3, "a": 0.3, "b": 0.3, "default": 0.15}


def draw_weights(raw: dict, seed: int, dtype: torch.dtype = torch.float32, scales: Optional[Dict[str, float]] = None,
                 shifts: Optional[Dict[str, float]] = None):
    """name -> tensor of the random model of ``raw`` and ``seed``. Norm weights of the layers and of the model's end
    are drawn around zero (the design adds one), gate biases and decay constants away from zero; ``scales``
    multiplies and ``shifts`` adds to named tensors (a name's last part stands for every layer's tensor)."""
    cfg = config_from_dict(raw)
    out = {}
    g = torch.Generator().manual_seed(seed)
    for d in declare_params(cfg.to_spec()):
        if d.optional:
            continue
        last = d.name.rsplit(".", 1)[-1]
        t = random_tensors([d], seed, torch.float32, std=STD.get(d.name if d.name in STD else last, STD["default"]))[d.name]
        if last in ("norm1", "norm2") or d.name == "final.norm":
            t = t - 1.0                                       # stored around zero
        elif d.name.endswith(".i.b"):
            t = torch.randn(d.shape, generator=g) * 0.5
        elif d.name.endswith(".f.b"):
            t = 2.0 + torch.randn(d.shape, generator=g) * 0.5  # forget gates near 0.9
        elif last == "A_log":
            t = torch.randn(d.shape, generator=g) * 0.5 - 1.0
        elif last == "dt_bias":
            t = torch.randn(d.shape, generator=g) * 0.5
        out[d.name] = t
    for table, f in ((scales, lambda t, v: t * v), (shifts, lambda t, v: t + v)):
        for name, v in (table or {}).items():
            hit = [n for n in out if n == name or n.endswith("." + name)]
            assert hit, name
            for n in hit:
                out[n] = f(out[n], v)
    return {n: t.to(dtype) for n, t in out.items()}


def make_folder(tmp_path, which: str, dtype: str = "bfloat16", scales=None, shifts=None, tag: str = "") -> str:
    raw, seed = CONFIGS[which]
    out = os.path.join(str(tmp_path), f"kobolix_{which}_{dtype}{tag}")
    if not os.path.isdir(out):
        os.makedirs(out)
        tdtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
        with open(os.path.join(out, "config.json"), "w", encoding="utf-8") as f:
            json.dump(raw, f, indent=1)
        write_safetensors(os.path.join(out, "model.safetensors"), draw_weights(raw, seed, tdtype, scales, shifts),
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
