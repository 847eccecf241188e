"""Parts that add to the token embedding before the first layer (registry "input").

An input part has ``declare_params(spec, hidden) -> [ParamDecl]``, ``__init__(spec, weights, hidden, dtype, device)``,
``state_need() -> StateNeed | None`` (per-request state of fixed size that the runner keeps for it) and
``add_to_stream(resid, batch, state)``, which adds its rows into the float stream of the step's tokens.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import kernels
from ..config.schema import InputSpec
from ..weights import MATRIX, ParamDecl
from .base import StateNeed
from .registry import register_input


@register_input("pair_hash")
class PairHashEmbedding:
    """A second embedding looked up by (previous token, token): row (previous * mul_prev + token * mul_cur)
    mod buckets of a [buckets + 1, width] table, the last row for a request's first token. The previous
    token of a portion's first token is the request's state: one int32 word a request slot on the device,
    read and then overwritten with the portion's last token by the kernel, so a step that takes its tokens
    from the device (a captured decode step chained to the one before) needs nothing from the host."""
    graph_safe = True

    @classmethod
    def declare_params(cls, spec: InputSpec, hidden: int) -> List[ParamDecl]:
        p = spec.params
        return [ParamDecl(spec.prefix + p.table_name, (p.buckets + 1, hidden), role=MATRIX)]

    def __init__(self, spec: InputSpec, weights: Dict[str, torch.Tensor], hidden: int, dtype: torch.dtype,
                 device: torch.device):
        p = spec.params
        self.buckets, self.mul_prev, self.mul_cur = int(p.buckets), int(p.mul_prev), int(p.mul_cur)
        self.table = weights[spec.prefix + p.table_name]

    def state_need(self) -> Optional[StateNeed]:
        return StateNeed((1,), torch.int32)

    def add_to_stream(self, resid: torch.Tensor, batch, state: torch.Tensor) -> None:
        kernels.current().pair_hash_add(resid, self.table, batch, state.view(-1), self.buckets, self.mul_prev,
                                        self.mul_cur)
