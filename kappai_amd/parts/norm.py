"""RMSNorm: ``y = x * 1/sqrt(mean(x^2) + eps) * w`` with eps inside the root
(kappai: src/backend/cpu/scalar/quants.c:1507-1512), computed in float32 and fused with the
residual sum that precedes it."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops, profile, tuning
from ..weights.spec import INIT_ONES, INIT_SMALL, VECTOR, TensorSpec
from .base import Norm, StreamUpdate, WeightedTerms, register_part
from .cdesc import FoldDesc


class RMSNorm(Norm):
    takes_partial_sums = True      # the kernel adds [S, T, width] partial sums itself, in order
    can_defer = True      # add_norm(..., defer=True) may hand out ops.ScaledRows or
                          # ops.FragmentRows in place of a tensor

    def __init__(self, name: str, width: int, eps: float, dtype: torch.dtype,
                 suffix: str = ".weight", weight_offset: float = 0.0, weight_scale: float = 1.0):
        """``suffix``: how the weight's tensor name ends in the checkpoint.  ``weight_offset``: the
        file stores the weight around zero and the norm multiplies by ``offset + w`` (1.0 for a
        "one plus" weight).  ``weight_scale``: a constant factor on the normalised rows that the
        owner wants folded in (a scale on the logits, for the norm before the head)."""
        self.name, self.width, self.eps, self.dtype = name, width, float(eps), dtype
        self.tensor_name = name + suffix
        self.weight_offset, self.weight_scale = float(weight_offset), float(weight_scale)
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        init = INIT_SMALL if self.weight_offset else INIT_ONES
        return [TensorSpec(self.tensor_name, (self.width,), VECTOR, init)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        w = tensors[self.tensor_name].to(torch.float32)
        if self.weight_offset or self.weight_scale != 1.0:
            w = (w + self.weight_offset) * self.weight_scale
        self.weight = w.contiguous()

    def norm_output(self, resid, y, rows_dtype=None, add: bool = True):
        """The norm on what a sublayer returned, added into the stream: ``resid += norm(y)`` in
        float32, in place (``add`` False: ``resid = norm(y)``).  ``y``: [T, width], float32
        partial sums [S, T, width], or ``WeightedTerms`` (two results and their weights, summed
        here).  Returns the new stream rounded to ``rows_dtype`` (None: nothing)."""
        a, sa, b, sb = y, 1.0, None, 1.0
        if isinstance(y, WeightedTerms):
            a, sa, b, sb = y.a, y.scale_a, y.b, y.scale_b
        with profile.scope("rmsnorm"):
            return ops.output_norm_add(resid, a, self.weight, self.eps, rows_dtype=rows_dtype,
                                       scale_a=sa, b=b, scale_b=sb, add=add)

    def fold(self):
        """(weight, eps) for a product that folds this norm in (``ops.AddInto``): the norm is
        ``x * weight / rms(x)``, so the product before it can hand on ``x * weight`` and the sums
        of squares, and the product after it divides."""
        return self.weight, self.eps

    def add_norm(self, resid, delta, rows=None, defer: bool = False):
        """``delta`` may also be what a product hands back that has added its result into
        ``resid`` itself: ``ops.Added``, or ``ops.ScaledRows`` made for this norm.  ``defer``: the
        caller's next part takes what the product kernels take in place of the rows: such
        ``ops.ScaledRows`` as they are, or ``ops.FragmentRows`` (8 to 16 rows, made here in the
        order the product loads them)."""
        if isinstance(delta, ops.Added):
            if (defer and rows is None and isinstance(delta, ops.ScaledRows)
                    and delta.weight is self.weight and delta.eps == self.eps
                    and delta.resid is resid):
                return delta
            delta = None             # the sum is in ``resid`` already
        n = resid.shape[0] if rows is None else rows.shape[0]
        fragment = (defer and tuning.FRAGMENT_ROWS and resid.is_cuda
                    and n >= tuning.FRAGMENT_ROWS_MIN
                    and ops.FragmentRows.fits(n, self.width, self.dtype)
                    and (delta is None or delta.dim() == 2 or delta.shape[0] <= 8))
        with profile.scope("rmsnorm" if rows is None else "logits_norm"):
            return ops.add_rmsnorm(resid, delta, self.weight, self.eps, self.dtype, rows=rows,
                                   write_resid=rows is None, fragment=fragment)

    def c_norm(self, plan):
        """The norm as the C side of a step runs it: the runner "norm.rms" reads weight and eps,
        which is also all a product needs to fold the norm in."""
        fold = plan.keep(FoldDesc(self.weight.data_ptr(), self.eps))
        return plan.norm("norm.rms", fold, fold=fold)

    def weight_bytes(self) -> int:
        return self.width * 4


register_part("norm", "rmsnorm", RMSNorm)


class LayerNorm(Norm):
    """``(x - mean) / sqrt(var + eps) * w`` without a bias (``var``: the mean of the squared
    deviations), in float32, in one kernel with the sum that precedes it.  The stream it reads may
    be kept in several copies [T, copies, width] (``read_streams``): the kernel then first gives
    the copies the update that is pending (``StreamUpdate``) and normalises their weighted sum."""

    takes_partial_sums = True      # the kernel adds [S, T, width] partial sums itself, in order

    def __init__(self, name: str, width: int, eps: float, dtype: torch.dtype, suffix: str = ""):
        self.name, self.width, self.eps, self.dtype = name, width, float(eps), dtype
        self.tensor_name = name + suffix
        self.weight: Optional[torch.Tensor] = None
        self._ones = {}

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.tensor_name, (self.width,), VECTOR, INIT_ONES)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.tensor_name].to(torch.float32).contiguous()

    def ones(self, *shape) -> torch.Tensor:
        """A float32 tensor of ones of this shape on the weight's device (made once)."""
        if shape not in self._ones:
            self._ones[shape] = torch.ones(shape, dtype=torch.float32, device=self.weight.device)
        return self._ones[shape]

    def read_streams(self, streams, in_w, pending: Optional[StreamUpdate] = None, source=None,
                     rows=None) -> torch.Tensor:
        """Normalised rows of ``sum_s in_w[s] x_s`` over the copies ``streams`` [T, S, width],
        after ``pending`` has been applied to them in place.  ``source`` [T, width]: the copies
        are made here, all equal to it.  ``rows``: only these rows (the copies keep their old
        values)."""
        S = streams.shape[1]
        with profile.scope("rmsnorm" if rows is None else "logits_norm"):
            return ops.hyper_step(
                streams, S, self.width, source=source,
                y=None if pending is None else pending.y,
                mix=None if pending is None else pending.mix,
                out_w=None if pending is None else pending.out, in_w=in_w, norm_w=self.weight,
                eps=self.eps, rows=rows, rows_dtype=self.dtype)

    def add_norm(self, resid, delta, rows=None):
        """The ``Norm`` interface on one stream [T, width]; or, on a stream in copies [T, S, width]
        with a pending ``StreamUpdate`` (or None), the norm of the copies' plain sum."""
        if isinstance(delta, ops.Added):
            delta = None
        if resid.dim() == 3:
            if delta is not None and not isinstance(delta, StreamUpdate):
                raise ValueError("a stream kept in copies takes its updates as StreamUpdate")
            return self.read_streams(resid, self.ones(resid.shape[1]), pending=delta, rows=rows)
        pending = None if delta is None else StreamUpdate(delta, self.ones(1, 1), self.ones(1))
        return self.read_streams(resid.unsqueeze(1), self.ones(1), pending=pending, rows=rows)

    def weight_bytes(self) -> int:
        return self.width * 4


register_part("norm", "layernorm", LayerNorm)
