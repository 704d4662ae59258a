"""A recurrent block around a real-gated linear unit.

Two branches of ``inner`` channels read the same rows: ``y = gelu_tanh(W_y h + b_y)`` and
``u = conv(W_x h + b_x)``, a causal convolution per channel over the last ``taps`` tokens with a
bias and no activation.  The channels are cut into ``blocks`` equal parts; in part b a square
matrix each makes the two gates, ``r = sigmoid(A_r[b] u_b + c_r[b])`` and
``i = sigmoid(A_i[b] u_b + c_i[b])``.  Per channel ``a = exp(-rate * r * softplus(lam))`` and

    S_t = a S_(t-1) + sqrt(1 - a^2) * i * u

from a zero state (the first token takes no other rule); the output is ``W_o (S * y)``.  Gates,
decays and the state are float32 (the gates' products keep their float32 sums); the state is a
slot of ``inner`` floats a request, and the convolution's last ``taps - 1`` inputs are state too.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from ..cache.specs import CacheBundle, FixedState
from ..kernels import ops, profile, tuning
from ..weights.spec import INIT_NORMAL, INIT_SMALL, MATRIX, VECTOR, TensorSpec
from .base import Mixer, register_part
from .linear import Linear
from .mingru import ScanChunks


class RealGatedUnit(Mixer):
    def __init__(self, prefix: str, width: int, inner: int, blocks: int, taps: int,
                 dtype: torch.dtype, rate: float = 8.0, names=None,
                 weight_suffix: str = ".weight", bias_suffix: str = ".bias"):
        n = {"y": "y", "x": "x", "conv": "conv", "r_gate": "ra", "i_gate": "ri", "lam": "lam",
             "o": "o"}
        n.update(names or {})
        if blocks < 1 or inner % blocks:
            raise ValueError(f"{prefix}: {inner} channels cannot be cut into {blocks} equal parts")
        if not 1 <= taps <= ops.CONV_SILU_MAX_TAPS:
            raise ValueError(f"{prefix}: {taps} taps; the kernel takes 1 to "
                             f"{ops.CONV_SILU_MAX_TAPS}")
        self.prefix, self.width, self.inner, self.dtype = prefix, width, inner, dtype
        self.blocks, self.taps, self.rate = int(blocks), int(taps), float(rate)
        self.inputs = Linear([prefix + n["x"], prefix + n["y"]], width, [inner, inner], bias=True,
                             stage="matmul_in_proj", weight_suffix=weight_suffix,
                             bias_suffix=bias_suffix)
        self.out = Linear([prefix + n["o"]], inner, [width], stage="matmul_out_proj",
                          weight_suffix=weight_suffix)
        self._conv = prefix + n["conv"] + weight_suffix
        self._conv_bias = prefix + n["conv"] + bias_suffix
        self._gates = [(prefix + n[k] + weight_suffix, prefix + n[k] + bias_suffix)
                       for k in ("r_gate", "i_gate")]
        self._lam = prefix + n["lam"]
        self.conv_taps = self.conv_bias = self.gate_w = self.gate_b = self.softplus_lam = None

    @property
    def step_tables(self) -> ScanChunks:
        return ScanChunks(tuning.SCAN_CHUNK_ROWS)

    def cache_spec(self):
        state = FixedState((self.inner,), "float32")
        if self.taps == 1:
            return state
        return CacheBundle((("state", state),
                            ("conv", FixedState((self.taps - 1, self.inner), "float32"))))

    def tensor_specs(self) -> List[TensorSpec]:
        part = self.inner // self.blocks
        specs = self.inputs.tensor_specs() + self.out.tensor_specs()
        specs += [TensorSpec(self._conv, (self.inner, self.taps), VECTOR, INIT_SMALL),
                  TensorSpec(self._conv_bias, (self.inner,), VECTOR, INIT_SMALL),
                  TensorSpec(self._lam, (self.inner,), VECTOR, INIT_SMALL)]
        for w, b in self._gates:
            specs += [TensorSpec(w, (self.blocks, part, part), MATRIX, INIT_NORMAL),
                      TensorSpec(b, (self.blocks, part), VECTOR, INIT_SMALL)]
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.inputs.bind(tensors)
        self.out.bind(tensors)
        self.conv_taps = tensors[self._conv].to(torch.float32).contiguous()
        self.conv_bias = tensors[self._conv_bias].to(torch.float32).contiguous()
        (wr, br), (wi, bi) = ((tensors[w], tensors[b]) for w, b in self._gates)
        # both gates of a block from one product: [blocks, r | i, part], biases laid out alike
        self.gate_w = torch.cat([wr, wi], dim=1).contiguous()
        self.gate_b = torch.cat([br.reshape(self.blocks, -1), bi.reshape(self.blocks, -1)],
                                dim=1).reshape(-1).to(torch.float32).contiguous()
        lam = tensors[self._lam].to(torch.float64)
        self.softplus_lam = torch.nn.functional.softplus(lam).to(torch.float32).contiguous()

    def forward(self, x, batch, cache, shared_cache: bool = False):
        if shared_cache:
            raise ValueError("a recurrent state cannot be read by another layer")
        C = self.inner
        proj = self.inputs.forward(x)                      # [T, x | y], biases added
        if self.taps > 1:
            state, conv_state = cache.part("state").state, cache.part("conv").state
        else:
            state = cache.state
            conv_state = torch.empty((state.shape[0], 0, C), dtype=torch.float32,
                                     device=state.device)
        if (batch.max_segment_rows == 1
                and C // self.blocks <= ops.GATED_UNIT_STEP_MAX_PART):
            # single rows: convolution, gates, recurrence and gated output in one kernel
            with profile.scope("scan"):
                y = ops.gated_unit_step(proj, self.conv_taps, self.conv_bias, conv_state,
                                        self.gate_w, self.gate_b, self.softplus_lam, self.rate,
                                        state, batch.seg_pos0, batch.seg_slot)
            return self.out.forward(y, partial_sums=True)
        with profile.scope("short_conv"):
            u = ops.conv_silu(proj, self.conv_taps, conv_state, batch.row_pos, batch.row_seg,
                              batch.seg_start, batch.seg_pos0, batch.seg_slot,
                              bias=self.conv_bias, activation=False)
        chunked = batch.max_segment_rows > tuning.SCAN_CHUNKS_FROM_ROWS
        with profile.scope("scan"):
            # (r | i) of every block before their sigmoid, float32 sums: a matrix a block
            gates = torch.empty((u.shape[0], 2 * C), dtype=torch.float32, device=u.device)
            part = C // self.blocks
            ops.headwise_linear(u, part, self.gate_w, out=gates, out_head_stride=2 * part,
                                out_dtype=torch.float32)
            y = ops.gated_unit_scan(
                gates, self.gate_b, u, proj[:, C:], self.softplus_lam, self.rate, state,
                batch.seg_start, batch.seg_pos0, batch.seg_slot,
                chunks=batch.extra.get("scan_chunks") if chunked else None,
                seg_chunk0=batch.extra.get("scan_seg_chunk0") if chunked else None,
                gate_part=part)
        return self.out.forward(y, partial_sums=True)

    def weight_bytes(self) -> int:
        return (self.inputs.weight_bytes() + self.out.weight_bytes()
                + self.gate_w.numel() * self.gate_w.element_size())


register_part("mixer", "real_gated_unit", RealGatedUnit)
