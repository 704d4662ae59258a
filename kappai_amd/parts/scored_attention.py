"""Softmax attention whose scores are worked on before the softmax, over the paged cache.

``q = W_q h``, ``k = W_k h``, ``v = W_v h``; q and k are each divided by the root mean square of
their WHOLE projection (all heads at once) and multiplied by a weight of that size; q is also
multiplied by ``1 + temp_coef * ln(floor((p + 1) / temp_every) + 1)`` at position p.  Then

    score(i, j) = softcap * tanh(q_i . k_j * scale / softcap) + rel[bucket(i - j), h]

over all ``j <= i`` (or the last ``window``; or, with ``chunk``, those ``j <= i`` with
``floor(j / chunk) = floor(i / chunk)``, chunks counted from position 0 of the sequence), a
softmax whose denominator also holds ``exp(sink[h])``, the weighted sum of the values, ``W_o``.
With ``position`` (a rotary encoding) the first places of every q and k head turn by the
position instead of the norm and the temperature; ``bias``: q, k and v have biases;
``values_from_keys``: there is no ``W_v``, a kv head's value is its key as projected, before the
rotation.  ``head_qk_norm``: every q and k head is divided by the root mean square of its own
``dim`` places and multiplied by a weight of that size which all heads share, before the
rotation.  ``sink_value``: the sink is this constant score for every head (0: a one in the
softmax's denominator) and no tensor.  ``head_gate``: a map ``W_g`` [heads, width] of the mixer's
input gives one number a head, and the head's result is multiplied by its sigmoid before ``W_o``.
``bucket``: a distance below half the
table's rows has a row of its own; larger ones share rows on a logarithmic scale that reaches the
last row at ``bias_max``.  Every piece is optional (``softcap`` 0, no table, no sink, no norm, no
temperature), so the part also serves designs that use some of them.

Queries, keys and values run through the framework's paged attention kernels as heads of one
size ``D`` that holds ``dim`` and ``vdim`` (``ops.projection_norm_store``); the table becomes a
bias by distance, one column a distance (``ops.ScoreMods``).
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import numpy as np
import torch

from ..cache.specs import PagedKV
from ..kernels import ops, profile, tuning
from ..weights.spec import INIT_ONES, INIT_SMALL, VECTOR, TensorSpec
from .attention import AttentionTiles
from .base import Mixer, register_part
from .linear import Linear


def log_distance_bucket(n: int, rows: int, far: float) -> int:
    """Row of the bias table for distance ``n``: ``n`` itself below ``rows // 2``, then
    logarithmic steps that reach the last row at distance ``far``."""
    half = rows // 2
    if n < half:
        return n
    if half == 0:
        return rows - 1
    step = math.log(n / half) / math.log(far / half) * (rows - half)
    return min(rows - 1, half + int(math.floor(step)))


def distance_bias_columns(table: torch.Tensor, far: float) -> torch.Tensor:
    """``table`` [rows, H] -> float32 [H, n]: column ``c`` is the bias at distance ``c``; the last
    column stands for every larger distance."""
    rows = table.shape[0]
    n = int(math.floor(far)) + 2
    idx = np.fromiter((log_distance_bucket(c, rows, far) for c in range(n)), dtype=np.int64,
                      count=n)
    return table.to(torch.float32)[torch.from_numpy(idx).to(table.device)].T.contiguous()


class ScoredAttention(Mixer):
    def __init__(self, prefix: str, width: int, num_heads: int, num_kv_heads: int, dim: int,
                 vdim: int, scale: float, dtype: torch.dtype, norm_eps: float = 0.0,
                 whole_qk_norm: bool = False, softcap: float = 0.0,
                 bias_buckets: int = 0, bias_far: float = 0.0, sink: bool = False,
                 temp_coef: float = 0.0, temp_every: int = 1, window: Optional[int] = None,
                 names=None, weight_suffix: str = ".weight", chunk: Optional[int] = None,
                 position=None, bias: bool = False, bias_suffix: str = ".bias",
                 values_from_keys: bool = False, head_qk_norm: bool = False,
                 sink_value: Optional[float] = None, head_gate: bool = False):
        n = {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm",
             "rel": "rel", "sink": "sink", "gate": "g"}
        n.update(names or {})
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads cannot be shared out over {num_kv_heads} kv heads")
        if bias_buckets and not bias_far > max(1.0, bias_buckets // 2):
            raise ValueError(f"{prefix}: the distance at which the bias table ends ({bias_far}) "
                             f"must lie beyond its linear half ({bias_buckets // 2})")
        self.prefix, self.width, self.dtype = prefix, width, dtype
        self.H, self.G, self.d, self.dv = num_heads, num_kv_heads, dim, vdim
        self.head_size = 16 * ((max(dim, vdim) + 15) // 16)
        self.scale, self.norm_eps, self.softcap = float(scale), float(norm_eps), float(softcap)
        self.whole_qk_norm = bool(whole_qk_norm)
        self.bias_buckets, self.bias_far, self.has_sink = int(bias_buckets), float(bias_far), sink
        self.temp_coef, self.temp_every = float(temp_coef), int(temp_every)
        self.window = int(window) if window else None
        self.chunk = int(chunk) if chunk else None
        if self.window and self.chunk:
            raise ValueError(f"{prefix}: a sliding window or chunks, not both")
        self.position, self.values_from_keys = position, bool(values_from_keys)
        self.head_qk_norm, self.head_gate = bool(head_qk_norm), bool(head_gate)
        self.sink_value = None if sink_value is None else float(sink_value)
        if self.head_qk_norm and (whole_qk_norm or temp_coef or self.values_from_keys):
            raise ValueError(f"{prefix}: the norm of every head by itself goes with neither the "
                             "whole-projection norm, the query temperature nor values that are "
                             "the keys")
        if self.sink_value is not None and sink:
            raise ValueError(f"{prefix}: a learned sink or a constant one, not both")
        if position is not None and (whole_qk_norm or temp_coef):
            raise ValueError(f"{prefix}: a rotation goes with neither the whole-projection norm "
                             "nor the query temperature")
        if position is not None and position.rot_dim > dim:
            raise ValueError(f"{prefix}: {position.rot_dim} places turn in heads of {dim}")
        if self.values_from_keys and vdim != dim:
            raise ValueError(f"{prefix}: values that are the keys have the keys' size {dim}, "
                             f"not {vdim}")
        stacked = ["q", "k"] + ([] if self.values_from_keys else ["v"])
        sizes = [num_heads * dim, num_kv_heads * dim] + (
            [] if self.values_from_keys else [num_kv_heads * vdim])
        self._gate_at = sum(sizes)          # where the gates' columns start in the projection
        if self.head_gate:
            stacked.append("gate")
            sizes.append(num_heads)
        self.qkv = Linear([prefix + n[k] for k in stacked], width, sizes, bias=bias,
                          stage="matmul_qkv", weight_suffix=weight_suffix,
                          bias_suffix=bias_suffix)
        self._o_name = prefix + n["o"] + weight_suffix
        self.out = Linear([prefix + n["o"]], num_heads * vdim, [width], stage="matmul_attn_out",
                          weight_suffix=weight_suffix)
        self._names = {k: prefix + n[k] for k in ("q_norm", "k_norm", "rel", "sink")}
        self.q_norm_w = self.k_norm_w = None
        self.mods = ops.ScoreMods()

    @property
    def step_tables(self) -> AttentionTiles:
        ok = (self.dtype == torch.bfloat16 and self.H // self.G <= 16 and self.head_size <= 256)
        return AttentionTiles(ops.ATTENTION_TILE_ROWS,
                              tuning.LONE_ROWS_FROM if ok and tuning.LONE_ROWS_FROM else None)

    def cache_spec(self):
        # (pages of chunks that lie behind stay with the request: only a window gives them back)
        return PagedKV(self.G, self.head_size, self.window)

    def tensor_specs(self) -> List[TensorSpec]:
        specs = self.qkv.tensor_specs() + self.out.tensor_specs()
        if self.whole_qk_norm:
            specs.append(TensorSpec(self._names["q_norm"], (self.H * self.d,), VECTOR, INIT_ONES))
            specs.append(TensorSpec(self._names["k_norm"], (self.G * self.d,), VECTOR, INIT_ONES))
        if self.head_qk_norm:
            specs.append(TensorSpec(self._names["q_norm"], (self.d,), VECTOR, INIT_ONES))
            specs.append(TensorSpec(self._names["k_norm"], (self.d,), VECTOR, INIT_ONES))
        if self.bias_buckets:
            specs.append(TensorSpec(self._names["rel"], (self.bias_buckets, self.H), VECTOR,
                                    INIT_SMALL))
        if self.has_sink:
            specs.append(TensorSpec(self._names["sink"], (self.H,), VECTOR, INIT_SMALL))
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.qkv.bind(tensors)
        H, dv, D = self.H, self.dv, self.head_size
        if D != dv:
            # the attention kernels hand back heads of D: the output map gets zero columns there
            w = tensors[self._o_name]
            wide = torch.zeros((w.shape[0], H, D), dtype=w.dtype, device=w.device)
            wide[:, :, :dv] = w.reshape(w.shape[0], H, dv)
            self.out.set_weight(wide.reshape(w.shape[0], H * D).contiguous())
        else:
            self.out.bind(tensors)
        if self.whole_qk_norm or self.head_qk_norm:
            self.q_norm_w = tensors[self._names["q_norm"]].to(torch.float32).contiguous()
            self.k_norm_w = tensors[self._names["k_norm"]].to(torch.float32).contiguous()
        bias = sink = None
        if self.bias_buckets:
            bias = distance_bias_columns(tensors[self._names["rel"]], self.bias_far)
        if self.has_sink:
            sink = tensors[self._names["sink"]].to(torch.float32).contiguous()
        elif self.sink_value is not None:
            sink = torch.full((H,), self.sink_value, dtype=torch.float32,
                              device=tensors[self._o_name].device)
        self.mods = ops.ScoreMods(self.softcap, bias, sink)

    def forward(self, x, batch, cache, shared_cache: bool = False):
        if shared_cache:
            raise ValueError("this attention does not read another layer's keys")
        H, G, D = self.H, self.G, self.head_size
        proj = self.qkv.forward(x)
        tables = batch.block_tables[cache.group]
        k_pool, v_pool = cache.pool("k"), cache.pool("v")
        with profile.scope("rope_kvput"):
            if self.head_qk_norm:
                rot = (self.position.rotation(x.device, batch.max_position)
                       if self.position is not None else None)
                q = ops.head_norm_rotate_store(
                    proj, H, G, self.d, self.dv, D, self.q_norm_w, self.k_norm_w, self.norm_eps,
                    rot.cos if rot else None, rot.sin if rot else None,
                    rot.rot_dim if rot else 0, rot.mode if rot else ops.ROT_NONE, k_pool, v_pool,
                    batch.row_pos, batch.row_seg, tables, cache.page_size)
            elif self.position is not None or self.values_from_keys:
                rot = (self.position.rotation(x.device, batch.max_position)
                       if self.position is not None else None)
                q = ops.rotate_widen_store(
                    proj, H, G, self.d, self.dv, D, rot.cos if rot else None,
                    rot.sin if rot else None, rot.rot_dim if rot else 0,
                    rot.mode if rot else ops.ROT_NONE, self.values_from_keys, k_pool, v_pool,
                    batch.row_pos, batch.row_seg, tables, cache.page_size)
            else:
                q = ops.projection_norm_store(
                    proj, H, G, self.d, self.dv, D, self.q_norm_w, self.k_norm_w, self.norm_eps,
                    self.temp_coef, self.temp_every, k_pool, v_pool, batch.row_pos,
                    batch.row_seg, tables, cache.page_size)
        with profile.scope("attn"):
            ctx = ops.paged_attention(q, H, G, D, k_pool, v_pool, batch.row_pos, batch.row_seg,
                                      tables, cache.page_size, self.scale,
                                      window=self.window or 0, chunk=self.chunk or 0,
                                      q_tiles=batch.extra.get("q_tiles"),
                                      single_rows=batch.max_segment_rows == 1,
                                      max_position=batch.max_position,
                                      lone_rows=batch.extra.get("lone_rows"),
                                      max_lone_position=batch.numbers.get("max_lone_position",
                                                                          -1),
                                      mods=self.mods)
            if self.head_gate:
                at = self._gate_at
                ops.sigmoid_gate(ctx, proj[:, at:at + H], D)
        return self.out.forward(ctx, partial_sums=True)

    def weight_bytes(self) -> int:
        return self.qkv.weight_bytes() + self.out.weight_bytes()


register_part("mixer", "scored_attention", ScoredAttention)
