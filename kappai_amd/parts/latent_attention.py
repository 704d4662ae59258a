"""Attention whose keys and values come from one low-rank latent per token.

``q = W_q h`` lies head by head as ``[dim unrotated | rot_dim rotated]``.  ``W_dkv h`` has
``rank + rot_dim`` rows: the first ``rank``, RMS-normed with a weight, are the latent ``c``; the
rest is a key part that is rotated by the position and shared by all heads.  Head h has the
unrotated key ``W_uk[h] c`` and the value ``W_uv[h] c``;

    score(i, j) = (q_un_i . W_uk[h] c_j + q_rot_i . k_rot_j) * scale

over the last ``window`` positions (None: all), a softmax whose denominator may hold
``exp(sink[h])``, then ``W_o`` on the heads' values side by side.  ``q_rank``: the queries come
through a latent of their own, ``q = W_uq n(W_dq h)`` with ``n`` an RMS norm with a weight.
``gate``: the heads' values side by side are multiplied, channel by channel, by
``sigmoid(W_g h)`` before ``W_o``.

Only ``c`` and the rotated part are kept per token.  ``q_un . W_uk c = (W_uk^T q_un) . c`` and
``sum_j p_j W_uv c_j = W_uv sum_j p_j c_j``: the queries are taken to the latent's space first
(``ops.headwise_linear``), the framework's paged attention kernels then see H query heads on ONE
kv head whose key is ``[c | rotated | 0]`` and whose value is ``c`` (``ops.latent_store``; heads of
one size D, a multiple of 16), and the heads' results are taken from the latent's space to
``vdim`` by a second product per head.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..cache.specs import PagedKV
from ..kernels import ops, profile, tuning
from ..weights.spec import INIT_NORMAL, INIT_ONES, INIT_SMALL, MATRIX, VECTOR, TensorSpec
from .attention import AttentionTiles
from .base import Mixer, PositionEncoding, register_part
from .linear import Linear


class LatentAttention(Mixer):
    def __init__(self, prefix: str, width: int, num_heads: int, dim: int, rot_dim: int, vdim: int,
                 rank: int, scale: float, norm_eps: float, dtype: torch.dtype,
                 position: Optional[PositionEncoding] = None, window: Optional[int] = None,
                 sink: bool = False, names=None, weight_suffix: str = ".weight",
                 q_rank: Optional[int] = None, gate: bool = False):
        """``position``: a rotary encoding over (part of) the ``rot_dim`` places, or None."""
        n = {"q": "q", "dkv": "dkv", "c_norm": "dkv.norm", "uk": "uk", "uv": "uv", "o": "o",
             "sink": "sink", "dq": "dq", "q_norm": "dq.norm", "uq": "uq", "gate": "g"}
        n.update(names or {})
        self.prefix, self.width, self.dtype = prefix, width, dtype
        self.H, self.d, self.rot, self.dv, self.r = num_heads, dim, rot_dim, vdim, rank
        self.head_size = 16 * ((rank + rot_dim + 15) // 16)
        self.scale, self.norm_eps = float(scale), float(norm_eps)
        self.window = int(window) if window else None
        self.position, self.has_sink = position, sink
        self.q_rank, self.has_gate = (int(q_rank) if q_rank else None), bool(gate)
        nq = num_heads * (dim + rot_dim)
        first, sizes = [prefix + n["q"], prefix + n["dkv"]], [nq, rank + rot_dim]
        self.up_q = None
        if self.q_rank:
            first[0], sizes[0] = prefix + n["dq"], self.q_rank
            self.up_q = Linear([prefix + n["uq"]], self.q_rank, [nq], stage="matmul_qkv",
                               weight_suffix=weight_suffix)
        if self.has_gate:
            first.append(prefix + n["gate"])
            sizes.append(num_heads * vdim)
        self._first_sizes = sizes
        self.q_dkv = Linear(first, width, sizes, stage="matmul_qkv", weight_suffix=weight_suffix)
        self._q_norm = prefix + n["q_norm"]
        self.q_norm_w = None
        self.out = Linear([prefix + n["o"]], num_heads * vdim, [width], stage="matmul_attn_out",
                          weight_suffix=weight_suffix)
        self._uk, self._uv = prefix + n["uk"] + weight_suffix, prefix + n["uv"] + weight_suffix
        self._c_norm, self._sink = prefix + n["c_norm"], prefix + n["sink"]
        self.to_latent = self.from_latent = self.c_norm_w = None
        self.mods = ops.ScoreMods()

    @property
    def step_tables(self) -> AttentionTiles:
        ok = self.dtype == torch.bfloat16 and self.H <= 16 and self.head_size <= 256
        return AttentionTiles(ops.ATTENTION_TILE_ROWS,
                              tuning.LONE_ROWS_FROM if ok and tuning.LONE_ROWS_FROM else None)

    def cache_spec(self):
        return PagedKV(1, self.head_size, self.window)

    def tensor_specs(self) -> List[TensorSpec]:
        specs = self.q_dkv.tensor_specs() + self.out.tensor_specs() + [
            TensorSpec(self._uk, (self.H * self.d, self.r), MATRIX, INIT_NORMAL),
            TensorSpec(self._uv, (self.H * self.dv, self.r), MATRIX, INIT_NORMAL),
            TensorSpec(self._c_norm, (self.r,), VECTOR, INIT_ONES)]
        if self.has_sink:
            specs.append(TensorSpec(self._sink, (self.H,), VECTOR, INIT_SMALL))
        if self.up_q is not None:
            specs += self.up_q.tensor_specs()
            specs.append(TensorSpec(self._q_norm, (self.q_rank,), VECTOR, INIT_ONES))
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.q_dkv.bind(tensors)
        self.out.bind(tensors)
        if self.up_q is not None:
            self.up_q.bind(tensors)
            self.q_norm_w = tensors[self._q_norm].to(torch.float32).contiguous()
        H, d, dv, r = self.H, self.d, self.dv, self.r
        # [H, out, in] each: to the latent's space (W_uk[h]^T) and from it (W_uv[h])
        self.to_latent = tensors[self._uk].reshape(H, d, r).transpose(1, 2).contiguous()
        self.from_latent = tensors[self._uv].reshape(H, dv, r).contiguous()
        self.c_norm_w = tensors[self._c_norm].to(torch.float32).contiguous()
        sink = tensors[self._sink].to(torch.float32).contiguous() if self.has_sink else None
        self.mods = ops.ScoreMods(0.0, None, sink)

    def forward(self, x, batch, cache, shared_cache: bool = False):
        if shared_cache:
            raise ValueError("this attention does not read another layer's keys")
        H, d, rot, r, D = self.H, self.d, self.rot, self.r, self.head_size
        proj = self.q_dkv.forward(x)
        nq = self._first_sizes[0]
        queries = proj
        if self.up_q is not None:
            # the queries' own latent: normed in float32, then up to the heads
            with profile.scope("rope_kvput"):
                cq = ops.rows_rmsnorm(proj, nq, self.q_norm_w, self.norm_eps)
            queries = self.up_q.forward(cq)
        rotn = self.position.rotation(x.device, batch.max_position) if self.position else None
        tables = batch.block_tables[cache.group]
        k_pool, v_pool = cache.pool("k"), cache.pool("v")
        with profile.scope("rope_kvput"):
            q = ops.latent_store(
                queries[:, :H * (d + rot)], proj[:, nq:nq + r + rot], H, d, rot, r, D,
                self.c_norm_w, self.norm_eps,
                rotn.cos if rotn else None, rotn.sin if rotn else None,
                rotn.rot_dim if rotn else 0, rotn.mode if rotn else ops.ROT_NONE, k_pool, v_pool,
                batch.row_pos, batch.row_seg, tables, cache.page_size)
            ops.headwise_linear(queries, d + rot, self.to_latent, out=q, out_head_stride=D)
        with profile.scope("attn"):
            ctx = ops.paged_attention(q, H, 1, D, k_pool, v_pool, batch.row_pos, batch.row_seg,
                                      tables, cache.page_size, self.scale,
                                      window=self.window or 0,
                                      q_tiles=batch.extra.get("q_tiles"),
                                      single_rows=batch.max_segment_rows == 1,
                                      max_position=batch.max_position,
                                      lone_rows=batch.extra.get("lone_rows"),
                                      max_lone_position=batch.numbers.get("max_lone_position",
                                                                          -1),
                                      mods=self.mods)
            at = nq + r + rot
            heads = ops.headwise_linear(
                ctx, D, self.from_latent,
                gate=proj[:, at:at + H * self.dv] if self.has_gate else None)
        return self.out.forward(heads, partial_sums=True)

    def weight_bytes(self) -> int:
        n = self.to_latent.numel() + self.from_latent.numel()
        up_q = self.up_q.weight_bytes() if self.up_q is not None else 0
        return (self.q_dkv.weight_bytes() + self.out.weight_bytes() + up_q
                + n * self.to_latent.element_size())


register_part("mixer", "latent_attention", LatentAttention)
