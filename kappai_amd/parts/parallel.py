"""Two mixers side by side: both read the same rows, and the result is
``left_scale * left(h) + right_scale * right(h)``.  The sum is left to whoever takes the result
(``parts.base.WeightedTerms``: a norm on the sublayer's output adds the two in float32 while it
normalises).  Each mixer keeps its own cache: the pair asks for a bundle with the members "left"
and "right" (a member that is a bundle itself is taken apart: "left.<name>").

``side_norms`` (two tensor names, with ``width`` and ``norm_eps``): each side's result is first
RMS-normed over the model width with a plain weight of its own,
``left_scale * n_l(left) + right_scale * n_r(right)``.  With side norms, or with ``summed``, the
pair adds its two sides itself in float32 (one kernel) and returns that update, which any norm
takes; an arrangement whose norm reads the mixer's input only needs this."""
from __future__ import annotations

from typing import Dict, List

import torch

from ..cache.manager import BundleView
from ..cache.specs import CacheBundle
from ..kernels import ops
from ..weights.spec import INIT_ONES, VECTOR, TensorSpec
from .base import Mixer, WeightedTerms, register_part


class ParallelMixer(Mixer):
    def __init__(self, left: Mixer, right: Mixer, left_scale: float = 1.0,
                 right_scale: float = 1.0, summed: bool = False, side_norms=None,
                 width: int = 0, norm_eps: float = 0.0):
        self.left, self.right = left, right
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)
        self.side_norms = tuple(side_norms) if side_norms else None
        if self.side_norms is not None and (len(self.side_norms) != 2 or width < 1):
            raise ValueError("side norms are two tensor names, and need the model width")
        self.summed = bool(summed) or self.side_norms is not None
        self.width, self.norm_eps = int(width), float(norm_eps)
        self.norm_w = (None, None)

    def _sides(self):
        return (("left", self.left), ("right", self.right))

    @property
    def capturable(self) -> bool:
        return self.left.capturable and self.right.capturable

    @property
    def step_tables(self):
        asked = []
        for _, m in self._sides():
            t = getattr(m, "step_tables", None)
            if t is not None:
                asked += list(t) if isinstance(t, (list, tuple)) else [t]
        return asked or None

    def cache_spec(self):
        members = []
        for side, m in self._sides():
            spec = m.cache_spec()
            if isinstance(spec, CacheBundle):
                members += [(f"{side}.{name}", s) for name, s in spec.parts]
            elif spec is not None:
                members.append((side, spec))
        return CacheBundle(tuple(members)) if members else None

    @staticmethod
    def _view(cache, side: str, mixer: Mixer):
        spec = mixer.cache_spec()
        if spec is None:
            return None
        if isinstance(spec, CacheBundle):
            return BundleView({name: cache.part(f"{side}.{name}") for name, _ in spec.parts})
        return cache.part(side)

    def tensor_specs(self) -> List[TensorSpec]:
        specs = self.left.tensor_specs() + self.right.tensor_specs()
        if self.side_norms is not None:
            specs += [TensorSpec(name, (self.width,), VECTOR, INIT_ONES)
                      for name in self.side_norms]
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.left.bind(tensors)
        self.right.bind(tensors)
        if self.side_norms is not None:
            self.norm_w = tuple(tensors[name].to(torch.float32).contiguous()
                                for name in self.side_norms)

    def forward(self, x, batch, cache, shared_cache: bool = False):
        if shared_cache:
            raise ValueError("a pair of mixers does not read another layer's cache")
        out = []
        for side, m in self._sides():
            y = m.forward(x, batch, self._view(cache, side, m))
            if isinstance(y, torch.Tensor) and y.dim() == 3:
                y = ops.sum_partial_sums(y)
            out.append(y)
        if out[0].dtype != out[1].dtype:
            out = [y if y.dtype == torch.float32 else ops.cast(y, torch.float32) for y in out]
        if self.summed:
            return ops.pair_norm_sum(out[0], out[1], self.left_scale, self.right_scale,
                                     self.norm_w[0], self.norm_w[1], self.norm_eps)
        return WeightedTerms(out[0], self.left_scale, out[1], self.right_scale)

    def weight_bytes(self) -> int:
        n = self.left.weight_bytes() + self.right.weight_bytes()
        return n + (8 * self.width if self.side_norms is not None else 0)


register_part("mixer", "parallel", ParallelMixer)
