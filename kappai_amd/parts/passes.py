"""What a pass over a run of layers starts with.

A model may run some of its layers several times in a row with the same weights, each pass with
caches of its own (``models.base.LayerCall`` names a block as often as it runs).  Right before
the first layer of pass ``t`` the stream takes, in this order, the embedded rows once more (every
pass but the first, when ``add_embedded``) and row ``t`` of a learned table [passes, width].
Everything is added in float32, together with the update the layer before left pending.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops, profile
from ..weights.spec import INIT_SMALL, VECTOR, TensorSpec
from .base import Hidden, Part, WeightedTerms


class PassEntry(Part):
    def __init__(self, table_name: Optional[str], n_passes: int, number: int, width: int,
                 add_embedded: bool):
        """``table_name``: the tensor [n_passes, width] whose row ``number`` is added (None: no
        row).  ``add_embedded``: the embedded rows are added before it."""
        if not 0 <= number < n_passes:
            raise ValueError(f"pass {number} of {n_passes}")
        self.table_name, self.n_passes, self.number = table_name, int(n_passes), int(number)
        self.width, self.add_embedded = int(width), bool(add_embedded)
        self.row: Optional[torch.Tensor] = None

    @property
    def reads_embedded(self) -> bool:
        return self.add_embedded

    def tensor_specs(self) -> List[TensorSpec]:
        if self.table_name is None:
            return []
        return [TensorSpec(self.table_name, (self.n_passes, self.width), VECTOR, INIT_SMALL)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        if self.table_name is not None:
            self.row = tensors[self.table_name][self.number].to(torch.float32).contiguous()

    def forward(self, h: Hidden, embedded: Optional[torch.Tensor], batch) -> Hidden:
        delta = h.delta
        if isinstance(delta, ops.Added):
            delta = None                       # a product has added its result already
        elif isinstance(delta, WeightedTerms):
            delta = ops.pair_norm_sum(delta.a, delta.b, delta.scale_a, delta.scale_b)
        elif isinstance(delta, torch.Tensor) and delta.dim() == 3:
            delta = ops.sum_partial_sums(delta)
        if self.add_embedded and embedded is None:
            raise ValueError("a pass that adds the embedded rows was given none")
        with profile.scope("rmsnorm"):
            ops.stream_enter(h.resid, delta, embedded if self.add_embedded else None, self.row)
        return Hidden(h.resid, None)

    def weight_bytes(self) -> int:
        return 4 * self.width if self.row is not None else 0
