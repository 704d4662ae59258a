"""Mixers whose memory is a matrix per head, ``S`` [dim, vdim] in float32, one slot a request.

``GatedLinearAttention``: ``q = W_q h * dim^-1/2``, ``k = W_k h``, ``v = W_v h``; a decay per key
channel ``a = sigmoid(z)^(1/tau)`` with ``z = W_a2 (W_a1 h) + b``; per head
``S <- diag(a) S + k v^T``, ``o = S^T q``; each head's ``o`` RMS-normed over ``vdim`` with a weight
shared by the heads, times ``silu(W_g h)``, then ``W_o``.

``GatedDeltaRule``: q, k ([kv_heads, dim]) and v ([heads, vdim]) pass a short causal convolution
per channel and SiLU; q and k become unit vectors per head (``x / sqrt(sum x^2 + 1e-6)``), q also
times ``dim^-1/2``; ``beta = sigmoid(W_b h)`` per head; a decay per head and key channel
``g = exp(-exp(A_log[h]) * softplus(W_a2 (W_a1 h) + dt_bias))``; per head ``S <- g S``,
``u = beta (v - S^T k)``, ``S <- S + k u^T``, ``o = S^T q`` (the read-out sees the token's own
write); each head's ``o`` divided by its root mean square, times a weight shared by the heads,
times ``sigmoid(W_g2 (W_g1 h))``, then ``W_o``.  The convolutions' last ``taps - 1`` inputs are
state as well.

``FixedDecayAttention``: ``q = silu(W_q h)``, ``k = silu(W_k h)``, ``v = silu(W_v h)``; one fixed
decay a head, ``S <- decay[h] S + k v^T``, ``o = S^T q`` with no other scale; the heads side by
side are RMS-normed TOGETHER with a weight [heads * vdim], times ``sigmoid(W_g h)``, then ``W_o``.

``BonusTimeMixing``: with ``h'`` the token before (zeros at position 0), each of r, k, v, g, w
reads its own mix ``h + (h' - h) * mu_s``; ``r, k, v = W_r, W_k, W_v`` of their mixes, the gate
``silu(W_g mix_g)``, a decay per head and key channel ``w = exp(-exp(W_w2 tanh(W_w1 mix_w) +
w0))``; per head ``o = (S + diag(u) k v^T)^T r`` (the bonus ``u`` [heads, dim] weighs the token
itself, which the state does not hold yet), then ``S <- diag(w) S + k v^T``; each head's ``o``
divided by its root mean square, times a weight [heads * dim] and the gate, then ``W_o``.  The
last row of ``h`` is state as well.

Projections, convolutions and their activations are stored in the compute dtype; decays,
softplus, exponentials, step sizes, unit vectors, the state and the per-head norm are float32.
"""
from __future__ import annotations

import math
from typing import Dict, List

import torch

from ..cache.specs import CacheBundle, FixedState
from ..kernels import ops, profile, tuning
from ..weights.spec import INIT_ONES, INIT_SMALL, VECTOR, TensorSpec
from .base import Mixer, register_part
from .linear import Linear
from .mingru import ScanChunks


def _columns(proj: torch.Tensor, start: int, n: int) -> torch.Tensor:
    """Columns ``start .. start + n`` of a product's result as the next product's input: a view
    when its rows start on 16 bytes, else a copy."""
    view = proj[:, start:start + n]
    if (view.data_ptr() % 16 or (proj.stride(0) * proj.element_size()) % 16) and proj.is_cuda:
        return view.contiguous()
    return view


class GatedLinearAttention(Mixer):
    def __init__(self, prefix: str, width: int, num_heads: int, dim: int, vdim: int, tau: float,
                 decay_rank: int, norm_eps: float, dtype: torch.dtype, names=None,
                 weight_suffix: str = ".weight", bias_suffix: str = ".bias"):
        n = {"q": "q", "k": "k", "v": "v", "g": "g", "a1": "a1", "a2": "a2", "norm": "norm",
             "o": "o"}
        n.update(names or {})
        self.prefix, self.width, self.dtype = prefix, width, dtype
        self.H, self.d, self.dv, self.rank = num_heads, dim, vdim, int(decay_rank)
        self.tau, self.norm_eps = float(tau), float(norm_eps)
        H, d, dv = num_heads, dim, vdim
        self.inputs = Linear([prefix + n[k] for k in ("q", "k", "v", "g", "a1")], width,
                             [H * d, H * d, H * dv, H * dv, self.rank], stage="matmul_in_proj",
                             weight_suffix=weight_suffix)
        self.decay = Linear([prefix + n["a2"]], self.rank, [H * d], stage="matmul_in_proj",
                            weight_suffix=weight_suffix)
        self.out = Linear([prefix + n["o"]], H * dv, [width], stage="matmul_out_proj",
                          weight_suffix=weight_suffix)
        self._decay_bias = prefix + n["a2"] + bias_suffix
        self._norm = prefix + n["norm"]
        self.decay_bias = self.norm_w = self.rate = None

    def cache_spec(self):
        return FixedState((self.H, self.dv, self.d), "float32")

    def tensor_specs(self) -> List[TensorSpec]:
        return (self.inputs.tensor_specs() + self.decay.tensor_specs() + self.out.tensor_specs()
                + [TensorSpec(self._decay_bias, (self.H * self.d,), VECTOR, INIT_SMALL),
                   TensorSpec(self._norm, (self.dv,), VECTOR, INIT_ONES)])

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for lin in (self.inputs, self.decay, self.out):
            lin.bind(tensors)
        self.decay_bias = tensors[self._decay_bias].to(torch.float32).contiguous()
        self.norm_w = tensors[self._norm].to(torch.float32).contiguous()
        # sigmoid(z)^(1/tau) = exp(-(1/tau) softplus(-z))
        self.rate = torch.full((self.H,), 1.0 / self.tau, dtype=torch.float32,
                               device=self.norm_w.device)

    def forward(self, x, batch, cache, shared_cache: bool = False):
        if shared_cache:
            raise ValueError("a recurrent state cannot be read by another layer")
        H, d, dv = self.H, self.d, self.dv
        proj = self.inputs.forward(x)
        o_k, o_v, o_g, o_a = H * d, 2 * H * d, 2 * H * d + H * dv, 2 * H * d + 2 * H * dv
        z = self.decay.forward(_columns(proj, o_a, self.rank))
        with profile.scope("scan"):
            o = ops.matrix_state_recurrence(
                proj, proj[:, o_k:], proj[:, o_v:], z, H, H, d, dv, self.rate, self.decay_bias,
                -1.0, d ** -0.5, cache.state, batch.seg_start, batch.seg_pos0, batch.seg_slot)
            y = ops.head_norm_gate(o, self.norm_w, self.norm_eps, proj[:, o_g:], ops.GATE_SILU,
                                   H, dv, self.dtype)
        return self.out.forward(y, partial_sums=True)

    def weight_bytes(self) -> int:
        return self.inputs.weight_bytes() + self.decay.weight_bytes() + self.out.weight_bytes()


register_part("mixer", "gated_linear_attention", GatedLinearAttention)


class FixedDecayAttention(Mixer):
    def __init__(self, prefix: str, width: int, num_heads: int, dim: int, vdim: int, decay,
                 norm_eps: float, dtype: torch.dtype, names=None, weight_suffix: str = ".weight"):
        n = {"q": "q", "k": "k", "v": "v", "g": "g", "norm": "norm", "o": "o"}
        n.update(names or {})
        decay = [float(a) for a in decay]
        if len(decay) != num_heads:
            raise ValueError(f"{prefix}: {len(decay)} decays for {num_heads} heads")
        if not all(0.0 <= a <= 1.0 for a in decay):
            raise ValueError(f"{prefix}: a decay lies between 0 and 1, got {decay}")
        self.prefix, self.width, self.dtype = prefix, width, dtype
        self.H, self.d, self.dv, self.decay = num_heads, dim, vdim, decay
        self.norm_eps = float(norm_eps)
        H, d, dv = num_heads, dim, vdim
        self.inputs = Linear([prefix + n[k] for k in ("q", "k", "v", "g")], width,
                             [H * d, H * d, H * dv, H * dv], stage="matmul_in_proj",
                             weight_suffix=weight_suffix)
        self.out = Linear([prefix + n["o"]], H * dv, [width], stage="matmul_out_proj",
                          weight_suffix=weight_suffix)
        self._norm = prefix + n["norm"]
        self.norm_w = self.rate = None

    @property
    def step_tables(self) -> ScanChunks:
        return ScanChunks(min(tuning.SCAN_CHUNK_ROWS, ops.FIXED_DECAY_CHUNK_ROWS))

    def cache_spec(self):
        return FixedState((self.H, self.dv, self.d), "float32")

    def tensor_specs(self) -> List[TensorSpec]:
        return (self.inputs.tensor_specs() + self.out.tensor_specs()
                + [TensorSpec(self._norm, (self.H * self.dv,), VECTOR, INIT_ONES)])

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.inputs.bind(tensors)
        self.out.bind(tensors)
        self.norm_w = tensors[self._norm].to(torch.float32).contiguous()
        self.rate = torch.tensor(self.decay, dtype=torch.float64).to(torch.float32).to(
            self.norm_w.device)

    def forward(self, x, batch, cache, shared_cache: bool = False):
        if shared_cache:
            raise ValueError("a recurrent state cannot be read by another layer")
        H, d, dv = self.H, self.d, self.dv
        proj = self.inputs.forward(x)
        o_k, o_v, o_g = H * d, 2 * H * d, 2 * H * d + H * dv
        # long portions: the decay is a constant, so a chunk of rows needs no chain along them
        chunked = batch.max_segment_rows > tuning.SCAN_CHUNKS_FROM_ROWS
        with profile.scope("scan"):
            o = ops.matrix_state_recurrence(
                proj, proj[:, o_k:], proj[:, o_v:], None, H, H, d, dv, self.rate, None, 1.0, 1.0,
                cache.state, batch.seg_start, batch.seg_pos0, batch.seg_slot, decay="fixed",
                silu_inputs=True,
                chunks=batch.extra.get("scan_chunks") if chunked else None,
                seg_chunk0=batch.extra.get("scan_seg_chunk0") if chunked else None,
                chunk_rows=min(tuning.SCAN_CHUNK_ROWS, ops.FIXED_DECAY_CHUNK_ROWS))
            # (all heads are normed together: one "head" of H * dv for the kernel)
            y = ops.head_norm_gate(o, self.norm_w, self.norm_eps, proj[:, o_g:],
                                   ops.GATE_SIGMOID, 1, H * dv, self.dtype)
        return self.out.forward(y, partial_sums=True)

    def weight_bytes(self) -> int:
        return self.inputs.weight_bytes() + self.out.weight_bytes()


register_part("mixer", "fixed_decay_attention", FixedDecayAttention)


class BonusTimeMixing(Mixer):
    MIXES = ("r", "k", "v", "g", "w")

    def __init__(self, prefix: str, width: int, num_heads: int, dim: int, decay_rank: int,
                 norm_eps: float, dtype: torch.dtype, names=None, weight_suffix: str = ".weight"):
        n = {"r": "r", "k": "k", "v": "v", "g": "g", "w1": "w1", "w2": "w2", "w0": "w0",
             "u": "u", "mu": "mu.", "norm": "norm", "o": "o"}
        n.update(names or {})
        self.prefix, self.width, self.dtype = prefix, width, dtype
        self.H, self.d, self.rank = num_heads, dim, int(decay_rank)
        self.norm_eps = float(norm_eps)
        H, d = num_heads, dim

        def lin(key, n_in, n_out, stage="matmul_in_proj"):
            return Linear([prefix + n[key]], n_in, [n_out], stage=stage,
                          weight_suffix=weight_suffix)

        self.r, self.k, self.v, self.g = (lin(s, width, H * d) for s in ("r", "k", "v", "g"))
        self.w1, self.w2 = lin("w1", width, self.rank), lin("w2", self.rank, H * d)
        self.out = lin("o", H * d, width, "matmul_out_proj")
        self._mu = [prefix + n["mu"] + s for s in self.MIXES]
        self._w0, self._u, self._norm = prefix + n["w0"], prefix + n["u"], prefix + n["norm"]
        self.mu = self.w0 = self.bonus = self.norm_w = None

    def _linears(self):
        return (self.r, self.k, self.v, self.g, self.w1, self.w2, self.out)

    @property
    def step_tables(self) -> ScanChunks:
        return ScanChunks(min(tuning.SCAN_CHUNK_ROWS, ops.FIXED_DECAY_CHUNK_ROWS))

    def cache_spec(self):
        return CacheBundle((("state", FixedState((self.H, self.d, self.d), "float32")),
                            ("shift", FixedState((self.width,), "float32"))))

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [s for lin in self._linears() for s in lin.tensor_specs()]
        specs += [TensorSpec(name, (self.width,), VECTOR, INIT_SMALL) for name in self._mu]
        specs += [TensorSpec(self._w0, (self.H * self.d,), VECTOR, INIT_SMALL),
                  TensorSpec(self._u, (self.H, self.d), VECTOR, INIT_SMALL),
                  TensorSpec(self._norm, (self.H * self.d,), VECTOR, INIT_ONES)]
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for lin in self._linears():
            lin.bind(tensors)
        self.mu = torch.stack([tensors[name].to(torch.float32) for name in self._mu]).contiguous()
        self.w0 = tensors[self._w0].to(torch.float32).contiguous()
        self.bonus = tensors[self._u].to(torch.float32).contiguous()
        self.norm_w = tensors[self._norm].to(torch.float32).reshape(self.H, self.d).contiguous()

    def forward(self, x, batch, cache, shared_cache: bool = False):
        if shared_cache:
            raise ValueError("a recurrent state cannot be read by another layer")
        H, d = self.H, self.d
        with profile.scope("short_conv"):
            mixes = ops.token_shift_mix(x, self.mu, cache.part("shift").state, batch.row_pos,
                                        batch.row_seg, batch.seg_start, batch.seg_slot)
        r, k, v, g = (lin.forward(mixes[i]) for i, lin in enumerate((self.r, self.k, self.v,
                                                                     self.g)))
        with profile.scope("ffn_act"):
            low = ops.tanh(self.w1.forward(mixes[4]))
        z = self.w2.forward(low)
        # long portions: chunk by chunk (the factors between two tokens are products of decays)
        chunked = batch.max_segment_rows > tuning.SCAN_CHUNKS_FROM_ROWS
        with profile.scope("scan"):
            o = ops.matrix_state_recurrence(
                r, k, v, z, H, H, d, d, None, self.w0, 1.0, 1.0, cache.part("state").state,
                batch.seg_start, batch.seg_pos0, batch.seg_slot, decay="double_exp",
                bonus=self.bonus,
                chunks=batch.extra.get("scan_chunks") if chunked else None,
                seg_chunk0=batch.extra.get("scan_seg_chunk0") if chunked else None,
                chunk_rows=min(tuning.SCAN_CHUNK_ROWS, ops.FIXED_DECAY_CHUNK_ROWS))
            y = ops.head_norm_gate(o, self.norm_w, self.norm_eps, g, ops.GATE_SILU, H, d,
                                   self.dtype)
        return self.out.forward(y, partial_sums=True)

    def weight_bytes(self) -> int:
        return sum(lin.weight_bytes() for lin in self._linears())


register_part("mixer", "bonus_time_mixing", BonusTimeMixing)


class GatedDeltaRule(Mixer):
    def __init__(self, prefix: str, width: int, num_heads: int, num_qk_heads: int, dim: int,
                 vdim: int, taps: int, decay_rank: int, gate_rank: int, norm_eps: float,
                 dtype: torch.dtype, unit_eps: float = 1e-6, names=None,
                 weight_suffix: str = ".weight"):
        n = {"q": "q", "k": "k", "v": "v", "b": "b", "a1": "a1", "a2": "a2", "g1": "g1",
             "g2": "g2", "o": "o", "conv": ".conv", "A_log": "A_log", "dt_bias": "dt_bias",
             "norm": "norm"}
        n.update(names or {})
        if num_heads % num_qk_heads:
            raise ValueError(f"{num_heads} heads cannot be shared out over {num_qk_heads} q/k heads")
        if not 1 <= taps <= ops.CONV_SILU_MAX_TAPS:
            raise ValueError(f"{prefix}: {taps} taps; the kernel takes 1 to "
                             f"{ops.CONV_SILU_MAX_TAPS}")
        self.prefix, self.width, self.dtype = prefix, width, dtype
        self.H, self.G, self.d, self.dv, self.taps = num_heads, num_qk_heads, dim, vdim, int(taps)
        self.ra, self.rg = int(decay_rank), int(gate_rank)
        self.norm_eps, self.unit_eps = float(norm_eps), float(unit_eps)
        H, G, d, dv = num_heads, num_qk_heads, dim, vdim
        self.channels = 2 * G * d + H * dv                 # what the convolution runs over
        # (the low-rank maps' inputs stand before the step sizes, whose count is any number)
        self.inputs = Linear([prefix + n[k] for k in ("q", "k", "v", "a1", "g1", "b")], width,
                             [G * d, G * d, H * dv, self.ra, self.rg, H], stage="matmul_in_proj",
                             weight_suffix=weight_suffix)
        self.decay = Linear([prefix + n["a2"]], self.ra, [H * d], stage="matmul_in_proj",
                            weight_suffix=weight_suffix)
        self.gate = Linear([prefix + n["g2"]], self.rg, [H * dv], stage="matmul_in_proj",
                           weight_suffix=weight_suffix)
        self.out = Linear([prefix + n["o"]], H * dv, [width], stage="matmul_out_proj",
                          weight_suffix=weight_suffix)
        self._conv = [(prefix + n[k] + n["conv"], c) for k, c in
                      (("q", G * d), ("k", G * d), ("v", H * dv))]
        self._a_log, self._dt_bias = prefix + n["A_log"], prefix + n["dt_bias"]
        self._norm = prefix + n["norm"]
        self.conv_taps = self.rate = self.dt_bias = self.norm_w = None

    def cache_spec(self):
        state = FixedState((self.H, self.dv, self.d), "float32")
        if self.taps == 1:
            return state
        return CacheBundle((("state", state),
                            ("conv", FixedState((self.taps - 1, self.channels), "float32"))))

    def tensor_specs(self) -> List[TensorSpec]:
        specs = (self.inputs.tensor_specs() + self.decay.tensor_specs() + self.gate.tensor_specs()
                 + self.out.tensor_specs())
        specs += [TensorSpec(name, (c, self.taps), VECTOR, INIT_SMALL) for name, c in self._conv]
        specs += [TensorSpec(self._a_log, (self.H,), VECTOR, INIT_SMALL),
                  TensorSpec(self._dt_bias, (self.H * self.d,), VECTOR, INIT_SMALL),
                  TensorSpec(self._norm, (self.dv,), VECTOR, INIT_ONES)]
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for lin in (self.inputs, self.decay, self.gate, self.out):
            lin.bind(tensors)
        self.conv_taps = torch.cat([tensors[name].to(torch.float32) for name, _ in self._conv],
                                   dim=0).contiguous()
        self.rate = torch.exp(tensors[self._a_log].to(torch.float32)).contiguous()
        self.dt_bias = tensors[self._dt_bias].to(torch.float32).contiguous()
        self.norm_w = tensors[self._norm].to(torch.float32).contiguous()

    def forward(self, x, batch, cache, shared_cache: bool = False):
        if shared_cache:
            raise ValueError("a recurrent state cannot be read by another layer")
        H, G, d, dv, C = self.H, self.G, self.d, self.dv, self.channels
        proj = self.inputs.forward(x)
        if self.taps > 1:
            state, conv_state = cache.part("state").state, cache.part("conv").state
        else:
            state = cache.state
            conv_state = torch.empty((state.shape[0], 0, C), dtype=torch.float32,
                                     device=state.device)
        with profile.scope("short_conv"):
            qkv = ops.conv_silu(proj, self.conv_taps, conv_state, batch.row_pos, batch.row_seg,
                                batch.seg_start, batch.seg_pos0, batch.seg_slot)
        z = self.decay.forward(_columns(proj, C, self.ra))
        gate = self.gate.forward(_columns(proj, C + self.ra, self.rg))
        with profile.scope("scan"):
            o = ops.matrix_state_recurrence(
                qkv, qkv[:, G * d:], qkv[:, 2 * G * d:], z, H, G, d, dv, self.rate, self.dt_bias,
                1.0, d ** -0.5, state, batch.seg_start, batch.seg_pos0, batch.seg_slot,
                beta=proj[:, C + self.ra + self.rg:], unit_qk=True, unit_eps=self.unit_eps)
            y = ops.head_norm_gate(o, self.norm_w, self.norm_eps, gate, ops.GATE_SIGMOID, H, dv,
                                   self.dtype)
        return self.out.forward(y, partial_sums=True)

    def weight_bytes(self) -> int:
        return sum(lin.weight_bytes() for lin in (self.inputs, self.decay, self.gate, self.out))


register_part("mixer", "gated_delta_rule", GatedDeltaRule)
