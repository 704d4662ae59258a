"""Mixture of experts: ``experts`` small gated feed-forward layers, of which every token uses
``top``.  Router logits ``W_router h`` in float32; the ``top`` largest are chosen and their
weights are the softmax over the chosen logits alone; the output is the weighted sum of the
chosen experts' ``W_down (silu(W_gate h) * W_up h)``.  Experts have no biases.  ``activation``
"relu_squared": the experts have no gate, ``W_down relu(W_up h)^2``.  ``router_bias``: a bias [E]
on the router's logits.  ``shared_hidden``: one more expert of that size and the same form
(``<prefix>shared.``) runs for every row, and its result is added with weight one.

The step's (row, choice) pairs are sorted by expert on the GPU and the experts' products run
over that order tile by tile, so nothing of the routing is read by the host.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops, profile, tuning
from ..weights.spec import INIT_NORMAL, INIT_SMALL, MATRIX, VECTOR, TensorSpec
from .base import FeedForward, register_part
from .linear import Linear


class MixtureOfExperts(FeedForward):
    def __init__(self, prefix: str, width: int, hidden: int, experts: int, top: int,
                 dtype: torch.dtype, names=None, weight_suffix: str = ".weight",
                 activation: str = "silu_gated", router_bias: bool = False,
                 shared_hidden: Optional[int] = None, bias_suffix: str = ".bias"):
        n = {"router": "router", "expert": "e{}.", "gate": "gate", "up": "up", "down": "down",
             "shared": "shared."}
        n.update(names or {})
        if activation not in ("silu_gated", "relu_squared"):
            raise ValueError(f"{prefix}: unknown expert activation {activation!r}; known: "
                             "silu_gated, relu_squared")
        if not 1 <= top <= min(experts, ops.MOE_MAX_TOP):
            raise ValueError(f"{prefix}: {top} of {experts} experts a token; the kernels take 1 to "
                             f"{ops.MOE_MAX_TOP}")
        self.prefix, self.width, self.hidden, self.dtype = prefix, width, hidden, dtype
        self.E, self.top = int(experts), int(top)
        self.gated = activation == "silu_gated"
        self._kinds = ("gate", "up", "down") if self.gated else ("up", "down")
        self._router = prefix + n["router"] + weight_suffix
        self._router_bias = prefix + n["router"] + bias_suffix if router_bias else None
        self._expert = [{k: prefix + n["expert"].format(e) + n[k] + weight_suffix
                         for k in self._kinds} for e in range(self.E)]
        self.router_bias: Optional[torch.Tensor] = None
        self.shared_up = self.shared_down = None
        if shared_hidden:
            if self.gated:
                raise ValueError(f"{prefix}: a shared expert goes with experts without a gate")
            sp = prefix + n["shared"]
            self.shared_up = Linear([sp + n["up"]], width, [int(shared_hidden)],
                                    stage="matmul_ffn_gate_up", weight_suffix=weight_suffix)
            self.shared_down = Linear([sp + n["down"]], int(shared_hidden), [width],
                                      stage="matmul_ffn_down", weight_suffix=weight_suffix)
        self.router: Optional[torch.Tensor] = None
        self.w_gate = self.w_up = self.w_down = None

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [TensorSpec(self._router, (self.E, self.width), MATRIX, INIT_NORMAL)]
        if self._router_bias:
            specs.append(TensorSpec(self._router_bias, (self.E,), VECTOR, INIT_SMALL))
        for names in self._expert:
            if self.gated:
                specs.append(TensorSpec(names["gate"], (self.hidden, self.width), MATRIX,
                                        INIT_NORMAL))
            specs.append(TensorSpec(names["up"], (self.hidden, self.width), MATRIX, INIT_NORMAL))
            specs.append(TensorSpec(names["down"], (self.width, self.hidden), MATRIX, INIT_NORMAL))
        if self.shared_up is not None:
            specs += self.shared_up.tensor_specs() + self.shared_down.tensor_specs()
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.router = tensors[self._router].to(torch.float32).contiguous()

        def stacked(key):
            w = torch.stack([tensors[names[key]].to(self.dtype) for names in self._expert]
                            ).contiguous()
            # bfloat16 matrices whose shape allows it are kept in the order the matrix-core
            # kernel loads them, and only so
            if w.is_cuda and tuning.FRAGMENT_ORDER and ops.ExpertFragments.fits(w):
                return ops.ExpertFragments.of(w)
            return w
        if self._router_bias:
            self.router_bias = tensors[self._router_bias].to(torch.float32).contiguous()
        self.w_gate = stacked("gate") if self.gated else None
        self.w_up = stacked("up")
        self.w_down = stacked("down")
        if self.shared_up is not None:
            self.shared_up.bind(tensors)
            self.shared_down.bind(tensors)

    def forward(self, x, batch):
        with profile.scope("router"):
            chosen, weights = ops.moe_route(x, self.router, self.top, bias=self.router_bias)
            plan = ops.moe_plan(chosen, self.E)
        also = None
        if self.shared_up is not None:
            hidden = self.shared_up.forward(x)
            with profile.scope("ffn_act"):
                hidden = ops.activate(hidden, ops.ACT_RELU_SQUARED)
            also = self.shared_down.forward(hidden, partial_sums=True)
        with profile.scope("matmul_ffn_gate_up", 0):
            act = (ops.moe_experts_gated(x, self.w_gate, self.w_up, plan) if self.gated
                   else ops.moe_experts_activated(x, self.w_up, plan))
        with profile.scope("matmul_ffn_down", 0):
            y = ops.moe_experts_down(act, self.w_down, plan)
            return ops.moe_combine(y, weights, plan, also=also)

    def weight_bytes(self) -> int:
        """What a step of one row reads: the router and ``top`` experts."""
        per_expert = len(self._kinds) * self.hidden * self.width * self.w_up.element_size()
        shared = 0
        if self.shared_up is not None:
            shared = self.shared_up.weight_bytes() + self.shared_down.weight_bytes()
        return self.router.numel() * 4 + self.top * per_expert + shared


register_part("feed_forward", "moe", MixtureOfExperts)
