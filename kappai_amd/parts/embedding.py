"""Token embedding and output head."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops, profile
from ..weights.spec import INIT_NORMAL, TABLE, TensorSpec
from .base import Part
from .linear import Linear


class TokenEmbedding(Part):
    """Rows of the table widened to float32, without a scale
    (kappai: src/recipe/scratch.c:195-235)."""

    def __init__(self, name: str, vocab: int, width: int, suffix: str = ".weight"):
        """``suffix``: how the table's tensor name ends in the checkpoint."""
        self.name, self.vocab, self.width = name, vocab, width
        self.tensor_name = name + suffix
        self.table: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.tensor_name, (self.vocab, self.width), TABLE, INIT_NORMAL)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.table = tensors[self.tensor_name]

    def forward(self, tokens: torch.Tensor) -> torch.Tensor:
        with profile.scope("embd"):
            return ops.embed_rows(tokens, self.table)

    def c_table(self):
        """The table as the C side of a step looks rows up in it."""
        return self.table

    def weight_bytes(self) -> int:
        return 0   # a step reads one row per token, not the table


class OutputHead(Part):
    """Logits in float32 for the rows asked for.  When tied the head is the embedding
    table itself (kappai: src/model.c:2562-2571)."""

    def __init__(self, name: str, vocab: int, width: int, tied_to: Optional[TokenEmbedding],
                 suffix: str = ".weight", softcap: float = 0.0):
        """``softcap`` c > 0: the logits leave as ``c * tanh(logits / c)``."""
        self.linear = Linear([name], width, [vocab], stage="logits_matmul", weight_suffix=suffix)
        self.tied_to = tied_to
        self.softcap = float(softcap)

    def tensor_specs(self) -> List[TensorSpec]:
        return [] if self.tied_to is not None else self.linear.tensor_specs()

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        if self.tied_to is not None:
            self.linear.bind_shared(self.tied_to.table)
            if isinstance(self.linear.weight, ops.InFragments):
                # one matrix, in the order the products read it: the embedding reads that too
                self.tied_to.table = self.linear.weight
        else:
            self.linear.bind(tensors)

    takes_deferred_rows = True     # a plain product: it takes what ops.linear takes

    def forward(self, x) -> torch.Tensor:
        logits = self.linear.forward(x, out_dtype=torch.float32)
        if self.softcap:
            with profile.scope("logits_matmul"):
                ops.softcap_rows(logits, self.softcap)
        return logits

    def c_linear(self):
        """The head's product as the C side of a step runs it (float32 logits)."""
        return self.linear

    def weight_bytes(self) -> int:
        return self.linear.weight_bytes()
