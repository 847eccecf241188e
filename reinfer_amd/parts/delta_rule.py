"""A gated delta rule as a token mixer: a float matrix state a head that is decayed, corrected towards the
token's value along its key, and read with its query.

q and k ([key_heads, key_dim]) and v ([heads, value_dim]) are projections of the mixer's input that pass a
short causal filter over time (a few taps a channel, zeros before a request's start) and silu; q and k are
then made unit vectors a head (q also times key_dim^-1/2). With beta_t = sigmoid(W_b h) and the decay
g_t = exp(-exp(A_log) softplus(W_a h + dt_bias)), both one number a head, value head a with its key head:

    S <- g_t S;   u = beta_t (v_t - S^T k_t);   S <- S + k_t u^T;   o_t = S^T q_t

so the read-out sees the token's own write. Each head's o is divided by its root mean square, multiplied by a
weight shared by the heads and by silu(W_g h), and W_o maps the heads back to the width. The filter, the
unit norms, the gates and the recurrence are float in either dtype. A request's state slot holds S in the
scan kernel's layout and, behind it, the last taps - 1 rows of the filter's input, so a prompt may be cut
anywhere.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from .. import kernels
from ..config.schema import MixerSpec
from ..weights import VECTOR, ParamDecl
from .base import LayerCache, StateNeed
from .registry import register_mixer


@register_mixer("gated_delta_rule")
class GatedDeltaRule:
    graph_safe = True       # the kernels read the step's shape from device arrays and leave state slot -1 alone

    @classmethod
    def declare_params(cls, spec: MixerSpec, prefix: str) -> List[ParamDecl]:
        p = spec.params
        H, G, dk, dv, w, taps = p.heads, p.key_heads, p.key_dim, p.value_dim, spec.hidden, p.conv_taps
        return [ParamDecl(prefix + "q", (G * dk, w)), ParamDecl(prefix + "q.conv", (G * dk, taps), role=VECTOR),
                ParamDecl(prefix + "k", (G * dk, w)), ParamDecl(prefix + "k.conv", (G * dk, taps), role=VECTOR),
                ParamDecl(prefix + "v", (H * dv, w)), ParamDecl(prefix + "v.conv", (H * dv, taps), role=VECTOR),
                ParamDecl(prefix + "b", (H, w)),
                ParamDecl(prefix + "A_log", (H,), init="zeros", role=VECTOR),
                ParamDecl(prefix + "norm", (dv,), init="norm", role=VECTOR),
                ParamDecl(prefix + "a", (H, w)),
                ParamDecl(prefix + "dt_bias", (H,), init="zeros", role=VECTOR),
                ParamDecl(prefix + "g", (H * dv, w)), ParamDecl(prefix + "o", (w, H * dv))]

    def __init__(self, spec: MixerSpec, weights: Dict[str, torch.Tensor], prefix: str, dtype: torch.dtype,
                 device: torch.device):
        p = spec.params
        if p is None:
            raise ValueError("gated_delta_rule: the sizes come in MixerSpec.params (DeltaRuleSpec)")
        if p.heads <= 0 or p.key_heads <= 0 or p.heads % p.key_heads:
            raise ValueError(f"gated_delta_rule: {p.heads} value heads do not divide into {p.key_heads} key heads")
        if p.conv_taps < 1:
            raise ValueError("gated_delta_rule: the filter has at least one tap")
        self.spec, self.dtype = spec, dtype
        self.heads, self.key_heads = int(p.heads), int(p.key_heads)
        self.key_dim, self.value_dim, self.taps = int(p.key_dim), int(p.value_dim), int(p.conv_taps)
        self.norm_eps, self.unit_eps = float(p.norm_eps), float(p.unit_eps)
        H, G, dk, dv = self.heads, self.key_heads, self.key_dim, self.value_dim
        # one product for [q | k | v | g]; the filter runs over the first three
        self.w_in = torch.cat([weights[prefix + n] for n in ("q", "k", "v", "g")], dim=0).contiguous()
        self.channels = 2 * G * dk + H * dv
        self.in_width = self.channels + H * dv
        self.filter = torch.cat([weights[prefix + n + ".conv"] for n in ("q", "k", "v")], dim=0).float().contiguous()
        # [b | a]: float results
        self.w_ba = torch.cat([weights[prefix + "b"], weights[prefix + "a"]], dim=0).contiguous()
        self.a_log = weights[prefix + "A_log"].float().contiguous()
        self.dt_bias = weights[prefix + "dt_bias"].float().contiguous()
        self.norm_weight = weights[prefix + "norm"].float().contiguous()
        self.w_o = weights[prefix + "o"]
        self.scan_floats = int(kernels.current().scan_state_floats("delta_rule", H, dk, dv))
        self.state_floats = self.scan_floats + (self.taps - 1) * self.channels

    def cache_need(self) -> StateNeed:
        return StateNeed((self.state_floats,), torch.float32)

    def forward(self, x, batch, cache: LayerCache):
        ops = kernels.current()
        T = x.shape[0]
        H, G, dk, dv = self.heads, self.key_heads, self.key_dim, self.value_dim
        proj = torch.empty((T, self.in_width), dtype=self.dtype, device=x.device)
        ops.linear(x, self.w_in, proj)
        ba = torch.empty((T, 2 * H), dtype=torch.float32, device=x.device)
        ops.linear(x, self.w_ba, ba)
        # filter + silu + unit norms -> float q | k | v; the filter's tail in the state moves on
        qkv = torch.empty((T, self.channels), dtype=torch.float32, device=x.device)
        ops.delta_rule_prepare(proj, self.filter, cache.state, self.scan_floats, batch, G, dk, H, dv, self.taps,
                               self.unit_eps, dk ** -0.5, qkv)
        read = torch.empty((T, H * dv), dtype=torch.float32, device=x.device)
        ops.delta_rule_scan(qkv, ba, self.a_log, self.dt_bias, cache.state, batch, H, G, dk, dv, read)
        act = torch.empty((T, H * dv), dtype=self.dtype, device=x.device)
        ops.head_norm_gate(read, self.norm_weight, False, proj[:, self.channels:], "silu", self.norm_eps, H, dv, act)
        out = torch.empty((T, self.spec.hidden), dtype=self.dtype, device=x.device)
        ops.linear(act, self.w_o, out)
        return out
