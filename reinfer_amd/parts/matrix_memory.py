"""A matrix memory with exponential gates (the mLSTM cell of xLSTM) as a token mixer.

Per head a state S [key_dim, value_dim], a normaliser n [key_dim] and a running maximum m of the log gates,
all float and all zero at a request's start. For token t, with q scaled by key_dim^-1/2, log input gate
a_t = cap tanh(z_i / cap) and log forget gate b_t = log sigmoid(cap tanh(z_f / cap)):

    m_t = max(b_t + m_{t-1}, a_t)
    S_t = exp(b_t + m_{t-1} - m_t) S_{t-1} + exp(a_t - m_t) k_t v_t^T        (n_t alike, with k_t alone)
    o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + denom_eps)

Each head's o is divided by its root mean square, the heads side by side are multiplied by a weight and by
sigmoid(W_g h), and W_o maps them back to the width. q, k, v and the gate's pre-activation come from one
product over the mixer's input; the two gate pre-activations a head from a second product that is
accumulated and kept in float. Everything from there to the read-out is float in either dtype; the state
lives in the request's state slot in the layout of the scan kernel (``scan_state_floats``), which walks a
request's tokens in order, the columns of S spread over lanes, waves and workgroups.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import kernels
from ..config.schema import MixerSpec
from ..weights import VECTOR, ParamDecl
from .base import LayerCache, StateNeed
from .registry import register_mixer


@register_mixer("matrix_memory")
class MatrixMemory:
    graph_safe = True       # the scan reads the step's shape from device arrays and leaves state slot -1 alone
    adds_scaled = True      # forward(..., resid=, resid_scale=) may add the output projection into the stream

    NAMES = ("q", "k", "v", "g", "o", "norm", "i", "i.b", "f", "f.b")

    @classmethod
    def declare_params(cls, spec: MixerSpec, prefix: str) -> List[ParamDecl]:
        p = spec.params
        H, dk, dv, w = p.heads, p.key_dim, p.value_dim, spec.hidden
        return [ParamDecl(prefix + "q", (H * dk, w)), ParamDecl(prefix + "k", (H * dk, w)),
                ParamDecl(prefix + "v", (H * dv, w)), ParamDecl(prefix + "g", (H * dv, w)),
                ParamDecl(prefix + "o", (w, H * dv)),
                ParamDecl(prefix + "norm", (H * dv,), init="norm", role=VECTOR),
                ParamDecl(prefix + "i", (H, w)), ParamDecl(prefix + "i.b", (H,), init="zeros", role=VECTOR),
                ParamDecl(prefix + "f", (H, w)), ParamDecl(prefix + "f.b", (H,), init="zeros", role=VECTOR)]

    def __init__(self, spec: MixerSpec, weights: Dict[str, torch.Tensor], prefix: str, dtype: torch.dtype,
                 device: torch.device):
        p = spec.params
        if p is None:
            raise ValueError("matrix_memory: the sizes come in MixerSpec.params (MatrixMemorySpec)")
        self.spec, self.dtype = spec, dtype
        self.heads, self.key_dim, self.value_dim = int(p.heads), int(p.key_dim), int(p.value_dim)
        self.gate_cap, self.norm_eps, self.denom_eps = float(p.gate_cap), float(p.norm_eps), float(p.denom_eps)
        H, dk, dv = self.heads, self.key_dim, self.value_dim
        # one product for everything that may be rounded to the compute dtype: [q | k | v | g]
        self.w_in = torch.cat([weights[prefix + n] for n in ("q", "k", "v", "g")], dim=0).contiguous()
        self.offsets = (0, H * dk, 2 * H * dk, 2 * H * dk + H * dv)
        self.in_width = 2 * H * dk + 2 * H * dv
        # the gates' pre-activations: [i | f], float results, float biases
        self.w_gates = torch.cat([weights[prefix + "i"], weights[prefix + "f"]], dim=0).contiguous()
        self.b_gates = torch.cat([weights[prefix + "i.b"], weights[prefix + "f.b"]], dim=0).float().contiguous()
        self.norm_weight = weights[prefix + "norm"].float().contiguous()
        self.w_o = weights[prefix + "o"]
        self.state_floats = int(kernels.current().scan_state_floats("matrix_memory", H, dk, dv))

    def cache_need(self) -> StateNeed:
        return StateNeed((self.state_floats,), torch.float32)

    def forward(self, x, batch, cache: LayerCache, resid: Optional[torch.Tensor] = None, resid_scale: float = 1.0):
        ops = kernels.current()
        T = x.shape[0]
        H, dk, dv = self.heads, self.key_dim, self.value_dim
        proj = torch.empty((T, self.in_width), dtype=self.dtype, device=x.device)
        ops.linear(x, self.w_in, proj)
        gates = torch.empty((T, 2 * H), dtype=torch.float32, device=x.device)
        ops.linear(x, self.w_gates, gates)
        read = torch.empty((T, H * dv), dtype=torch.float32, device=x.device)
        ops.matrix_memory_scan(proj, self.offsets[0], self.offsets[1], self.offsets[2], gates, self.b_gates,
                               cache.state, batch, H, dk, dv, self.gate_cap, dk ** -0.5, self.denom_eps, read)
        act = torch.empty((T, H * dv), dtype=self.dtype, device=x.device)
        ops.head_norm_gate(read, self.norm_weight, True, proj[:, self.offsets[3]:], "sigmoid", self.norm_eps,
                           H, dv, act)
        can_add = getattr(ops, "can_accumulate", None)
        if resid is not None and can_add and can_add(act, self.w_o):
            ops.linear_skinny(act, self.w_o, resid, accumulate=True, alpha=resid_scale)     # x += s * act . Wo^T
            return None
        out = torch.empty((T, self.spec.hidden), dtype=self.dtype, device=x.device)
        ops.linear(act, self.w_o, out)
        return out
