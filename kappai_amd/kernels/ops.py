"""Python faces of the HIP kernels.

Each function checks on the host that shapes, dtypes, strides and devices are what the
kernel and its grid assume, then launches on torch's current HIP stream.  Tensors must
live on the GPU; nothing here computes on the CPU.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Optional

import torch

from .lib import check, library

F32, BF16, I32 = torch.float32, torch.bfloat16, torch.int32
MAX_HEAD_DIM = 512
MAX_GRID_Y = 65535
DECODE_WAVES = 4096       # blocks the grid of the split-key decode attention provides for: the
                          # kernel itself aims at half as many at work, counting the keys the
                          # rows really hold (requests of mixed lengths get shorter splits)
DECODE_MAX_SPLITS = 128   # partial results of a row's head that the merge kernel adds up at most
# Keys up to which one block a (row, kv head) takes them all, its waves merging in LDS (8 requests
# at 200 keys: 7.4 us against 9.4 for the split kernel and its merge; even at 1024 keys, and from
# there on the split kernel wins: 22 against 35 us at 4096 keys, a wave taking its chunks one
# after the other where the split kernel has a wave for each)
DECODE_BLOCK_MAX_KEYS = 512

_c_int, _c_float, _c_long, _vp = ctypes.c_int, ctypes.c_float, ctypes.c_long, ctypes.c_void_p


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> _vp:
    """The current stream of the current device, as the handle the kernels' launchers take."""
    if _raw_stream is not None:         # the same value without building a Stream object
        return _vp(_raw_stream(torch.cuda.current_device()))
    return _vp(torch.cuda.current_stream().cuda_stream)


def _ptr(t: Optional[torch.Tensor]) -> _vp:
    return _vp(0 if t is None else t.data_ptr())


def _need(cond: bool, msg) -> None:
    """``msg`` is the text or a function that makes it (the text is then only put together
    when the check fails: these checks run for every kernel of every step)."""
    if not cond:
        raise ValueError(msg() if callable(msg) else msg)


def _gpu(name: str, t: torch.Tensor, dtype=None, contiguous=True) -> None:
    if not isinstance(t, torch.Tensor):
        raise ValueError(f"{name}: a tensor is needed")
    if not t.is_cuda:
        raise ValueError(f"{name}: must live on the GPU (kappai_amd has no CPU path), "
                         f"got {t.device}")
    if dtype is not None and t.dtype is not dtype:
        dts = dtype if isinstance(dtype, (tuple, list)) else (dtype,)
        if t.dtype not in dts:
            raise ValueError(f"{name}: dtype {t.dtype}, expected {' or '.join(map(str, dts))}")
    if contiguous and not t.is_contiguous():
        raise ValueError(f"{name}: must be contiguous")


def _is_bf16(dtype) -> int:
    _need(dtype in (F32, BF16), lambda: f"compute dtype must be float32 or bfloat16, got {dtype}")
    return 1 if dtype == BF16 else 0


# ---------------------------------------------------------------------------------------
def embed_rows(ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """float32 [T, D] rows of ``table`` ([V, D], float32 or bfloat16, or ``InFragments``: a tied
    output head's matrix) at ``ids`` (int32)."""
    _gpu("ids", ids, I32)
    kind = 2 if isinstance(table, InFragments) else None
    if kind is None:
        _gpu("table", table, (F32, BF16))
        kind = _is_bf16(table.dtype)
    _need(ids.dim() == 1 and table.dim() == 2, "embed_rows: ids [T], table [V, D]")
    T, D = ids.shape[0], table.shape[1]
    out = torch.empty((T, D), dtype=F32, device=table.device)
    check(library("elementwise").kappai_embed_rows(
        _ptr(ids), _ptr(table), _c_int(kind), _ptr(out), _c_int(T), _c_int(D),
        _stream()), "embed_rows")
    return out


def embed_rmsnorm(ids: torch.Tensor, table: torch.Tensor, weight: torch.Tensor, eps: float,
                  out_dtype, fragment: bool = False):
    """``embed_rows`` and the RMSNorm of its rows in one kernel: (float32 rows [T, D], the
    normalised rows as ``add_rmsnorm`` would return them), the same bits as the two kernels.  For
    widths that are multiples of 8 up to 8192 (of 32 for a table in fragment order)."""
    _gpu("ids", ids, I32)
    _gpu("weight", weight, F32)
    kind = 2 if isinstance(table, InFragments) else None
    if kind is None:
        _gpu("table", table, (F32, BF16))
        kind = _is_bf16(table.dtype)
    _need(ids.dim() == 1 and table.dim() == 2, "embed_rmsnorm: ids [T], table [V, D]")
    T, D = ids.shape[0], table.shape[1]
    _need(weight.shape == (D,), lambda: f"embed_rmsnorm: weight {tuple(weight.shape)} for D={D}")
    _need(D % 8 == 0 and D <= 8192 and (kind != 2 or D % 32 == 0),
          lambda: f"embed_rmsnorm: a width of {D} takes embed_rows and add_rmsnorm")
    if fragment:
        _need(FragmentRows.fits(T, D, out_dtype),
              "embed_rmsnorm: rows in fragment order need bfloat16, at most 16 rows and a width "
              "that is a multiple of 32 (up to 8192)")
    resid = torch.empty((T, D), dtype=F32, device=weight.device)
    out = torch.empty((16 if fragment else T, D), dtype=out_dtype, device=weight.device)
    check(library("elementwise").kappai_embed_rmsnorm(
        _ptr(ids), _ptr(table), _c_int(kind), _ptr(resid), _ptr(weight), _ptr(out), _c_int(T),
        _c_int(D), _c_float(eps), _c_int(_is_bf16(out_dtype)), _c_int(1 if fragment else 0),
        _stream()), "embed_rmsnorm")
    return resid, (FragmentRows(out, T, resid) if fragment else out)


def place_tokens(tokens: torch.Tensor, dst_rows: torch.Tensor, chosen: torch.Tensor,
                 src_idx: torch.Tensor) -> None:
    """``tokens[dst_rows[i]] = chosen[src_idx[i]]`` (all int32, on the GPU): token ids that
    sampling kernels left on the GPU go into a step's token table.  The host vouches for the
    indices (rows of this step, places in ``chosen``)."""
    for name, t in (("tokens", tokens), ("dst_rows", dst_rows), ("chosen", chosen),
                    ("src_idx", src_idx)):
        _gpu(name, t, I32)
        _need(t.dim() == 1, lambda: f"place_tokens: {name} must have one dimension")
    _need(dst_rows.shape == src_idx.shape, "place_tokens: as many rows as places")
    check(library("elementwise").kappai_place_tokens(
        _ptr(tokens), _ptr(dst_rows), _ptr(chosen), _ptr(src_idx), _c_int(dst_rows.shape[0]),
        _stream()), "place_tokens")


def tokens_to_host(src: torch.Tensor, dst: torch.Tensor) -> None:
    """The int32 values of ``src`` (on the GPU) into ``dst``, pinned host memory of at least as
    many, written by a kernel: they are there once an event recorded behind this call has
    happened.  Unlike a copy command towards the host, this does not make the host wait when it
    queues the next copy towards the GPU."""
    _gpu("src", src, I32)
    _need(isinstance(dst, torch.Tensor) and not dst.is_cuda and dst.is_pinned()
          and dst.dtype is I32 and dst.is_contiguous(),
          "tokens_to_host: dst must be contiguous pinned host memory of int32")
    n = src.numel()
    _need(dst.numel() >= n, lambda: f"tokens_to_host: {n} values for {dst.numel()} places")
    check(library("elementwise").kappai_copy_ints(
        ctypes.c_void_p(dst.data_ptr()), _ptr(src), _c_int(n), _stream()), "tokens_to_host")


def ints_from_host(src: torch.Tensor, dst: torch.Tensor) -> None:
    """The int32 values of ``src`` (pinned host memory, written by the host before this call)
    into ``dst`` on the GPU, read by a kernel: the tables of a step go this way, so that a step
    is kernels only and the host never waits inside a copy command while steps are queued
    ahead."""
    _gpu("dst", dst, I32)
    _need(isinstance(src, torch.Tensor) and not src.is_cuda and src.is_pinned()
          and src.dtype is I32 and src.is_contiguous(),
          "ints_from_host: src must be contiguous pinned host memory of int32")
    n = src.numel()
    _need(dst.numel() >= n, lambda: f"ints_from_host: {n} values for {dst.numel()} places")
    check(library("elementwise").kappai_copy_ints(
        _ptr(dst), ctypes.c_void_p(src.data_ptr()), _c_int(n), _stream()), "ints_from_host")


def add_rmsnorm(resid: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor,
                eps: float, out_dtype, rows: Optional[torch.Tensor] = None,
                write_resid: bool = True, fragment: bool = False):
    """RMSNorm of ``resid (+ delta)``; with ``write_resid`` the sum replaces ``resid``.
    ``delta`` is [T, D] in the compute dtype, or float32 partial sums [S, T, D] (a product
    split over K) that are added in order.  ``rows`` (int32) picks the rows to normalise; the
    result then has one row per entry.  ``fragment`` (at most 16 rows of bfloat16, a width that is
    a multiple of 32): the rows come back as ``FragmentRows``, in the order in which the product
    kernel for 1 to 16 rows loads them."""
    _gpu("resid", resid, F32)
    _gpu("weight", weight, F32)
    _need(resid.dim() == 2 and weight.shape == (resid.shape[1],),
          lambda: f"add_rmsnorm: resid {tuple(resid.shape)} and weight {tuple(weight.shape)} "
                  "disagree")
    isb = _is_bf16(out_dtype)
    n_part, pstride, delta_f32 = 1, 0, 0
    if delta is not None:
        if delta.dim() == 3:
            _gpu("delta", delta, F32)
            _need(delta.shape[1:] == resid.shape, "add_rmsnorm: partial sums must be [S, T, D]")
            n_part, pstride, delta_f32 = delta.shape[0], resid.numel(), 1
        else:
            _gpu("delta", delta, (out_dtype, F32))
            _need(delta.shape == resid.shape, "add_rmsnorm: delta must have resid's shape")
            delta_f32 = 1 if delta.dtype == F32 else 0
    n = resid.shape[0]
    if rows is not None:
        _gpu("rows", rows, I32)
        _need(not (write_resid and delta is not None),
              "add_rmsnorm: a row selection cannot update the residual")
        n = rows.shape[0]
    D = resid.shape[1]
    if fragment:
        _need(FragmentRows.fits(n, D, out_dtype) and n_part <= 8,
              "add_rmsnorm: rows in fragment order need bfloat16, at most 16 rows and a width "
              "that is a multiple of 32 (up to 8192)")
    out = torch.empty((16 if fragment else n, D), dtype=out_dtype, device=resid.device)
    check(library("elementwise").kappai_add_rmsnorm(
        _ptr(resid), _ptr(delta), _c_int(delta_f32), _c_int(n_part), _c_long(pstride), _ptr(weight),
        _ptr(out), _ptr(rows), _c_int(n), _c_int(D), _c_float(eps),
        _c_int(1 if write_resid else 0), _c_int(isb), _c_int(1 if fragment else 0), _stream()),
        "add_rmsnorm")
    return FragmentRows(out, n, resid) if fragment else out


FRAGMENT_ROWS_FROM = 8     # from this many rows on, rows for the next product go in fragment order


class FragmentRows:
    """At most 16 normalised rows [n, D] of a decode step, stored in the order in which the
    product kernel for 1 to 16 rows loads its activations ([D / 32][(k % 32) / 8][16 rows][8
    values], see ``fragment_order`` for the matrices): a load instruction of that kernel then
    touches whole cache lines of neighbouring rows instead of half a line of every row.
    ``linear``, ``linear_swiglu`` and ``linear_shortconv_step`` take it in place of the rows;
    ``materialize`` gives the rows as an ordinary tensor.  ``resid_after`` is the residual the
    norm has updated (the interface of ``ScaledRows``, so that a part takes either)."""

    def __init__(self, data: torch.Tensor, n_rows: int, resid: torch.Tensor):
        self.data, self.resid_after = data, resid
        self.shape = torch.Size((n_rows, data.shape[1]))
        self.device, self.dtype = data.device, data.dtype

    @staticmethod
    def fits(n_rows: int, width: int, out_dtype) -> bool:
        return out_dtype == BF16 and 1 <= n_rows <= 16 and width % 32 == 0 and width <= 8192

    def materialize(self) -> torch.Tensor:
        n, D = self.shape
        out = torch.empty((n, D), dtype=self.dtype, device=self.device)
        check(library("elementwise").kappai_rows_from_fragments(
            _ptr(self.data), _ptr(out), _c_int(n), _c_int(D), _stream()), "rows_from_fragments")
        return out


FUSED_MAX_ROWS = 16        # rows of a decode step whose products fold norm and residual sum in


class Added:
    """What a product hands back when it has added its result into the residual stream itself
    (``AddInto``): there is no update left to add.  ``resid`` is the stream it added to."""

    def __init__(self, resid: torch.Tensor):
        self.resid = resid


class ScaledRows(Added):
    """At most 16 rows of a decode step, on their way from a product that added its result into
    the residual stream (``AddInto`` with a norm weight) to the product after the RMSNorm that
    follows: ``data`` holds bf16(resid * weight), not yet divided by the rows' root mean square
    ([n, D], or 16 rows in fragment order), and ``ss`` [parts, 16] the sums of resid^2 over ranges
    of columns (row m at [:, m]; the columns beyond n hold nothing).  ``linear``, ``linear_swiglu`` and ``linear_shortconv_step`` take it in place of
    the normalised rows and scale their results by 1 / sqrt(sum of the parts / D + eps), which is
    the same product (RMSNorm(x) W^T = (x * w) W^T / rms(x)) without a kernel in between.
    ``materialize`` runs the ordinary norm kernel on the residual instead.  ``resid_after`` is
    the residual to go on with (the interface of ``FragmentRows``)."""

    def __init__(self, data: torch.Tensor, n_rows: int, fragment: bool, ss: torch.Tensor,
                 weight: torch.Tensor, eps: float, resid: torch.Tensor):
        super().__init__(resid)
        self.data, self.fragment, self.ss, self.weight, self.eps = data, fragment, ss, weight, eps
        self.resid_after = resid
        self.shape = torch.Size((n_rows, resid.shape[1]))
        self.device, self.dtype = data.device, data.dtype

    def materialize(self) -> torch.Tensor:
        return add_rmsnorm(self.resid, None, self.weight, self.eps, self.dtype)

    def _scale_args(self):
        return (_ptr(self.ss), _c_int(self.ss.shape[0]), _c_float(self.eps))


_NO_SCALE = (_vp(0), _c_int(0), _c_float(0.0))


class AddInto:
    """Asks a product to add its result into ``resid`` (float32 [M, N], in place, in float32)
    instead of returning it (kappai fuses the residual sum into the product the same way,
    src/recipe/graph_passes.c:135-163).  With ``norm_weight`` (and ``eps``) the RMSNorm that follows
    is folded in as well: the product hands back ``ScaledRows`` for the product after that norm.
    A product that cannot do it (more than 16 rows, float32 weights, ...) returns its result as
    always, and the caller goes on as without this."""

    def __init__(self, resid: torch.Tensor, norm_weight: Optional[torch.Tensor] = None,
                 eps: float = 0.0):
        self.resid, self.norm_weight, self.eps = resid, norm_weight, float(eps)


def add_residual(resid: torch.Tensor, delta: torch.Tensor) -> None:
    _gpu("resid", resid, F32)
    _gpu("delta", delta, (F32, BF16))
    _need(delta.shape == resid.shape, "add_residual: shapes differ")
    check(library("elementwise").kappai_add_residual(
        _ptr(resid), _ptr(delta), _c_long(resid.numel()), _c_int(_is_bf16(delta.dtype)),
        _stream()), "add_residual")


def sum_partial_sums(parts: torch.Tensor) -> torch.Tensor:
    """float32 [T, D] from the partial sums [S, T, D] of a product split over K, added in order:
    for a consumer (a norm, a block) that takes a plain update only."""
    _gpu("parts", parts, F32)
    _need(parts.dim() == 3, "sum_partial_sums: [S, T, D] is needed")
    out = torch.empty(parts.shape[1:], dtype=F32, device=parts.device)
    check(library("elementwise").kappai_sum_partials(
        _ptr(parts), _c_int(parts.shape[0]), _c_long(out.numel()), _ptr(out), _stream()),
        "sum_partials")
    return out


def stream_read(buf: torch.Tensor, blocks: int = 0) -> int:
    """Launches one plain read of ``buf`` (a kernel that only loads) and returns the bytes it
    reads: the yardstick for the kernels that stream weights and cache.  ``blocks``: how many
    blocks of four waves share the read (0: 512)."""
    _gpu("buf", buf)
    n = ctypes.c_long(0)
    check(library("elementwise").kappai_stream_read(
        _ptr(buf), _c_long(buf.numel() * buf.element_size()), _vp(0), ctypes.byref(n),
        _c_int(blocks), _stream()), "stream_read")
    return n.value


def mfma_probe(iters: int = 20000, device="cuda:0") -> float:
    """Launches a kernel that only issues bfloat16 matrix instructions from registers and returns
    the floating-point operations it performs: the yardstick for the products of prompt steps."""
    out = torch.empty(1024 * 256, dtype=F32, device=device)
    flops = ctypes.c_double(0.0)
    check(library("elementwise").kappai_mfma_probe(
        _ptr(out), _c_int(iters), ctypes.byref(flops), _stream()), "mfma_probe")
    return flops.value


def swiglu(gate_up: torch.Tensor) -> torch.Tensor:
    """``silu(gate_up[:, :F]) * gate_up[:, F:]`` for a fused [T, 2F] projection."""
    _gpu("gate_up", gate_up, (F32, BF16))
    _need(gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0, "swiglu: [T, 2F] is needed")
    T, F = gate_up.shape[0], gate_up.shape[1] // 2
    out = torch.empty((T, F), dtype=gate_up.dtype, device=gate_up.device)
    check(library("elementwise").kappai_swiglu(
        _ptr(gate_up), _ptr(out), _c_int(T), _c_int(F), _c_int(_is_bf16(gate_up.dtype)),
        _stream()), "swiglu")
    return out


def tanh(x: torch.Tensor) -> torch.Tensor:
    """``tanh`` of every element, stored as ``x`` is."""
    _gpu("x", x, (F32, BF16))
    out = torch.empty_like(x)
    check(library("elementwise").kappai_unary(
        _ptr(x), _ptr(out), _c_long(x.numel()), _c_int(0), _c_int(_is_bf16(x.dtype)), _stream()),
        "tanh")
    return out


def cast(x: torch.Tensor, dtype) -> torch.Tensor:
    _gpu("x", x, (F32, BF16))
    if x.dtype == dtype:
        return x
    out = torch.empty(x.shape, dtype=dtype, device=x.device)
    check(library("elementwise").kappai_cast(
        _ptr(x), _ptr(out), _c_long(x.numel()), _c_int(_is_bf16(x.dtype)),
        _c_int(_is_bf16(dtype)), _stream()), "cast")
    return out


# ---------------------------------------------------------------------------------------
def fragment_order(weight: torch.Tensor) -> Optional[torch.Tensor]:
    """A copy of a bfloat16 matrix [N, K] in the order in which the product kernel for 1 to 16
    rows loads it: pieces of 16 rows x 32 of K, each laid out lane by lane ([N / 16][K / 32]
    [(k % 32) / 8][row % 16][8 values]), so that one load instruction of a wave reads 1 KB in
    one piece.  None when the shape does not allow it (N a multiple of 16, K of 32).  Every
    product kernel for bfloat16 reads a matrix in this order (the kernels for few rows 10-20 %
    faster than rows, the block kernels for prompts as fast: a tile's 64 of K of 16 rows are
    2 KB in two pieces instead of 16 pieces of 128 bytes), so a matrix is kept in this order
    only: ``InFragments``."""
    if weight.dtype != BF16 or weight.dim() != 2:
        return None
    N, K = weight.shape
    if N % 16 or K % 32 or N == 0:
        return None
    return (weight.contiguous().view(N // 16, 16, K // 32, 4, 8).permute(0, 2, 3, 1, 4)
            .contiguous().view(N, K))


class InFragments:
    """A bfloat16 matrix [N, K] of which only ``fragment_order(matrix)`` is kept.  ``linear``,
    ``linear_swiglu``, ``linear_shortconv_step`` and ``embed_rows`` take it in place of the
    matrix; it has the matrix's ``shape`` and ``dtype``.  ``rows(n)``: its first ``n`` rows (a
    multiple of 16), sharing the memory."""

    def __init__(self, data: torch.Tensor):
        _gpu("fragments", data, BF16)
        _need(data.dim() == 2 and data.shape[0] % 16 == 0 and data.shape[1] % 32 == 0
              and data.data_ptr() % 16 == 0,
              lambda: f"fragments: [N, K] with N a multiple of 16 and K of 32, got {tuple(data.shape)}")
        self.data = data
        self.shape, self.dtype, self.device = data.shape, data.dtype, data.device

    @classmethod
    def of(cls, weight: torch.Tensor) -> Optional["InFragments"]:
        """``weight`` in fragment order, or None when its shape or dtype does not allow it."""
        frag = fragment_order(weight) if weight.is_cuda else None
        return None if frag is None else cls(frag)

    def dim(self) -> int:
        return 2

    def data_ptr(self) -> int:
        return self.data.data_ptr()

    def numel(self) -> int:
        return self.data.numel()

    def element_size(self) -> int:
        return self.data.element_size()

    def rows(self, n: int) -> "InFragments":
        _need(0 < n <= self.shape[0] and n % 16 == 0, lambda: f"fragments: the first {n} rows")
        return InFragments(self.data[:n])

    def materialize(self) -> torch.Tensor:
        """The matrix as rows again (for tests and tools; a copy made by torch)."""
        N, K = self.shape
        return (self.data.view(N // 16, K // 32, 4, 16, 8).permute(0, 3, 1, 2, 4)
                .reshape(N, K).contiguous())


def _matrix(weight, weight_frag: Optional[torch.Tensor]):
    """The two addresses the product kernels take: (the matrix as rows or null, the matrix in
    fragment order or null)."""
    if isinstance(weight, InFragments):
        _need(weight_frag is None, "a matrix kept in fragment order has no second copy")
        return _vp(0), _vp(weight.data.data_ptr())
    if weight_frag is None:
        return _vp(weight.data_ptr()), _vp(0)
    _gpu("weight_frag", weight_frag, BF16)
    _need(weight_frag.shape == weight.shape and weight.shape[0] % 16 == 0
          and weight.shape[1] % 32 == 0 and weight_frag.data_ptr() % 16 == 0,
          "weight_frag: the fragment-order copy must have the matrix's shape [N, K] with N a "
          "multiple of 16 and K of 32")
    return _vp(weight.data_ptr()), _vp(weight_frag.data_ptr())


def _gpu_matrix(name: str, weight, dtype) -> None:
    if not isinstance(weight, InFragments):
        _gpu(name, weight, dtype)


def split_k_for(M: int, N: int, K: int) -> int:
    """How many K ranges a product is cut into when its consumer takes partial sums (1: not
    split).  Decode (M <= 64): so that about 512 blocks stream the matrix (17 rows and more: what
    suits the kernel that takes them).  Larger M: the number that a model of the block kernel's
    time likes best (a product with few blocks is bound by the length of K and gains from being
    cut until the chip is full or the float partial sums cost more than the cut saves).  The rule
    itself lives beside the C side's step (``csrc/engine.hip``), which asks it as well."""
    return int(library("engine").kappai_split_k_for(_c_int(M), _c_int(N), _c_int(K)))


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
           out_dtype=None, force_kernel: int = 0, partial_sums: bool = False,
           split_k: Optional[int] = None,
           weight_frag: Optional[torch.Tensor] = None,
           add_into: Optional[AddInto] = None):
    """``x [M, K] @ weight[N, K]^T (+ bias)``.  A bfloat16 matrix runs on the matrix cores
    with float accumulation; a float32 matrix runs in true 32-bit arithmetic, whatever the
    activations' dtype.  ``x`` may be a view with a row stride.  With ``partial_sums`` the
    result may come back as float32 [S, M, N], the sums over S ranges of K, for a consumer
    that adds them (a matrix with few columns is then streamed by enough blocks).  ``x`` may
    be ``ScaledRows`` or ``FragmentRows``.  ``weight`` may be ``InFragments`` (a bfloat16 matrix
    kept in fragment order only); or ``weight_frag`` (``fragment_order(weight)``) may come beside
    the rows, which the kernels that are faster with it read.  ``add_into``: see ``AddInto``; the
    result is then ``Added`` or ``ScaledRows`` when the product could add its result itself."""
    a_frag = 0
    scale = None
    if isinstance(x, ScaledRows):
        if (weight.dtype != BF16 or force_kernel not in (0, 2) or weight.dim() != 2
                or weight.shape[1] != x.shape[1] or weight.data_ptr() % 16
                or weight.shape[1] % 8):
            x = x.materialize()          # only the kernel for 1 to 16 rows scales its results
        else:
            scale, partial_sums = x, False          # its kernel keeps K in one piece
            if x.fragment:
                a_frag, n_frag, x = 1, x.shape[0], x.data
            else:
                x = x.data
    if isinstance(x, FragmentRows):
        if (weight.dtype != BF16 or force_kernel not in (0, 2) or weight.dim() != 2
                or weight.shape[1] != x.shape[1] or weight.data_ptr() % 16):
            x = x.materialize()
        else:
            a_frag, n_frag, x = 1, x.shape[0], x.data     # 16 row slots, n_frag of them filled
    _gpu("x", x, (F32, BF16), contiguous=False)
    _gpu_matrix("weight", weight, (F32, BF16))
    _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1],
          lambda: f"linear: x {tuple(x.shape)} does not meet weight {tuple(weight.shape)}")
    _need(x.stride(1) == 1 or x.shape[1] == 1, "linear: x must have unit stride along K")
    M, K = x.shape
    if a_frag:
        M = n_frag
    N = weight.shape[0]
    out_dtype = out_dtype or x.dtype
    if bias is not None:
        _gpu("bias", bias, F32)
        _need(bias.shape == (N,), lambda: f"linear: bias {tuple(bias.shape)} for N={N}")
    if weight.dtype == F32:
        xf = x if x.dtype == F32 else cast(x.contiguous(), F32)
        out = torch.empty((M, N), dtype=F32, device=x.device)
        check(library("gemm").kappai_gemm_f32(
            _ptr(xf), _ptr(weight), _ptr(bias), _ptr(out), _c_int(M), _c_int(N), _c_int(K),
            _c_int(xf.stride(0) if M > 1 else K), _c_int(N), _stream()), "gemm_f32")
        return out if out_dtype == F32 else cast(out, out_dtype)
    xb = x if x.dtype == BF16 else cast(x.contiguous(), BF16)
    lda = xb.stride(0) if M > 1 else K
    if not (K % 8 == 0 and lda % 8 == 0 and xb.data_ptr() % 16 == 0
            and weight.data_ptr() % 16 == 0):
        # the matrix-core kernels read 16 bytes at a time; anything else goes the plain way
        _need(scale is None, "linear: scaled rows reached the plain kernel")
        _need(not force_kernel,
              lambda: f"linear: K ({K}) and the row stride ({lda}) must be multiples of 8 and "
                      "the tensors 16-byte aligned for the kernel that was asked for")
        _need(M <= MAX_GRID_Y, lambda: f"linear: {M} rows with a width that is no multiple of 8")
        _need(not isinstance(weight, InFragments),
              "linear: a matrix kept in fragment order needs 16-byte aligned rows of x")
        out = torch.empty((M, N), dtype=out_dtype, device=x.device)
        check(library("gemm").kappai_gemm_bf16_any(
            _ptr(xb), _ptr(weight), _ptr(bias), _ptr(out), _c_int(M), _c_int(N), _c_int(K),
            _c_int(lda), _c_int(N), _c_int(0 if out_dtype == BF16 else 1), _stream()),
            "gemm_bf16_any")
        return out
    scale_args = scale._scale_args() if scale is not None else _NO_SCALE
    if (add_into is not None and M <= FUSED_MAX_ROWS and force_kernel in (0, 2)
            and add_into.resid.dtype == F32 and add_into.resid.is_contiguous()
            and tuple(add_into.resid.shape) == (M, N)):
        # the result joins the residual stream inside the kernel
        resid, nw = add_into.resid, add_into.norm_weight
        _gpu("resid", resid, F32)
        rows = ss = None
        fragment = False
        if nw is not None:
            _gpu("norm_weight", nw, F32)
            _need(nw.shape == (N,), lambda: f"linear: norm weight {tuple(nw.shape)} for N={N}")
            fragment = FRAGMENT_ROWS_FROM <= M and FragmentRows.fits(M, N, BF16)
            rows = torch.empty((16 if fragment else M, N), dtype=BF16, device=x.device)
            ss = torch.empty(((N + 7) // 8, 16), dtype=F32, device=x.device)
        check(library("gemm").kappai_gemm_bf16(
            _ptr(xb), *_matrix(weight, weight_frag), _ptr(bias), _vp(0), _c_int(M),
            _c_int(N), _c_int(K), _c_int(lda), _c_int(N), _c_int(1), _c_int(force_kernel),
            _c_int(1), _c_int(a_frag), *scale_args, _ptr(resid), _c_int(resid.stride(0)),
            _ptr(nw), _ptr(rows), _c_int(1 if fragment else 0), _ptr(ss), _stream()),
            "gemm_bf16 (into the residual)")
        if nw is None:
            return Added(resid)
        return ScaledRows(rows, M, fragment, ss, nw, add_into.eps, resid)
    ksplit = (split_k or split_k_for(M, N, K)) if partial_sums else 1
    if ksplit > 1:
        out = torch.empty((ksplit, M, N), dtype=F32, device=x.device)
        out_is_f32 = 1
    else:
        out = torch.empty((M, N), dtype=out_dtype, device=x.device)
        out_is_f32 = 0 if out_dtype == BF16 else 1
    check(library("gemm").kappai_gemm_bf16(
        _ptr(xb), *_matrix(weight, weight_frag), _ptr(bias), _ptr(out), _c_int(M),
        _c_int(N), _c_int(K),
        _c_int(lda), _c_int(N), _c_int(out_is_f32), _c_int(force_kernel), _c_int(ksplit),
        _c_int(a_frag), *scale_args, _vp(0), _c_int(0), _vp(0), _vp(0), _c_int(0), _vp(0),
        _stream()), "gemm_bf16")
    return out


SWIGLU_GROUP = 16     # gate and up rows alternate in groups of this many rows


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """The layout ``linear_swiglu`` reads: 16 gate rows, the 16 up rows of the same columns, the
    next 16 gate rows, ...  [2F, K] from two [F, K] matrices; F must be a multiple of 16."""
    F, K = gate.shape
    _need(up.shape == gate.shape and F % SWIGLU_GROUP == 0,
          lambda: f"interleave_gate_up: {tuple(gate.shape)} and {tuple(up.shape)}; F must be a "
                  f"multiple of {SWIGLU_GROUP}")
    g = gate.reshape(F // SWIGLU_GROUP, 1, SWIGLU_GROUP, K)
    u = up.reshape(F // SWIGLU_GROUP, 1, SWIGLU_GROUP, K)
    return torch.cat([g, u], dim=1).reshape(2 * F, K).contiguous()


def _out_in_fragment_order(wanted: bool, M: int, N: int, force_kernel: int) -> bool:
    return (wanted and FRAGMENT_ROWS_FROM <= M <= FUSED_MAX_ROWS and N % 32 == 0
            and force_kernel in (0, 2))


def linear_swiglu(x: torch.Tensor, weight: torch.Tensor, force_kernel: int = 0,
                  weight_frag: Optional[torch.Tensor] = None, out_fragment: bool = False,
                  activation: int = 0):
    """``silu(x Wg^T) * (x Wu^T)`` in one kernel: ``weight`` [2F, K] holds the gate and up
    matrices interleaved by ``interleave_gate_up``; bfloat16 only.  Returns [M, F].  ``x`` may
    be ``ScaledRows`` or ``FragmentRows``.  ``out_fragment``: with 8 to 16 rows the result may
    come back as ``FragmentRows`` for the product that follows.  ``activation``: ``GLU_SILU`` (0)
    or ``GLU_GELU_TANH`` (1) in place of silu; the product kernels are built once per gate."""
    scale = None
    if isinstance(x, ScaledRows):
        if (force_kernel not in (0, 2) or weight.dtype != BF16 or weight.dim() != 2
                or weight.shape[1] != x.shape[1] or weight.shape[0] % (2 * SWIGLU_GROUP)
                or weight.data_ptr() % 16 or weight.shape[1] % 8):
            x = x.materialize()
        else:
            scale = x
            x = FragmentRows(x.data, x.shape[0], x.resid) if x.fragment else x.data
    a_frag, n_frag = 0, 0
    if isinstance(x, FragmentRows):
        if force_kernel not in (0, 2) or weight.dim() != 2 or weight.shape[1] != x.shape[1]:
            x = x.materialize()
        else:
            a_frag, n_frag, x = 1, x.shape[0], x.data
    _gpu("x", x, BF16, contiguous=False)
    _gpu_matrix("weight", weight, BF16)
    _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1]
          and weight.shape[0] % (2 * SWIGLU_GROUP) == 0,
          lambda: f"linear_swiglu: x {tuple(x.shape)}, weight {tuple(weight.shape)}")
    _need(x.stride(1) == 1 or x.shape[1] == 1, "linear_swiglu: x must have unit stride along K")
    M, K = x.shape
    if a_frag:
        M = n_frag
    F = weight.shape[0] // 2
    lda = x.stride(0) if M > 1 else K
    _need(K % 8 == 0 and lda % 8 == 0 and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0,
          lambda: f"linear_swiglu: K ({K}) and the row stride ({lda}) must be multiples of 8 "
                  "and the tensors 16-byte aligned")
    c_frag = _out_in_fragment_order(out_fragment, M, F, force_kernel)
    out = torch.empty((16 if c_frag else M, F), dtype=BF16, device=x.device)
    gemm = library("gemm") if not activation else library("gemm", GATE_ACT=int(activation))
    check(gemm.kappai_gemm_bf16_swiglu(
        _ptr(x), *_matrix(weight, weight_frag), _ptr(out), _c_int(M), _c_int(F), _c_int(K),
        _c_int(lda), _c_int(F),
        _c_int(force_kernel), _c_int(a_frag),
        *(scale._scale_args() if scale is not None else _NO_SCALE), _c_int(1 if c_frag else 0),
        _stream()), "gemm_bf16_swiglu")
    return FragmentRows(out, M, None) if c_frag else out


def linear_shortconv_step(x: torch.Tensor, in_proj: torch.Tensor, in_bias: Optional[torch.Tensor],
                          taps: torch.Tensor, conv_bias: Optional[torch.Tensor],
                          state: torch.Tensor, seg_pos0: torch.Tensor,
                          seg_slot: torch.Tensor,
                          weight_frag: Optional[torch.Tensor] = None,
                          out_fragment: bool = False):
    """A conv layer's decode step in one kernel, for a batch in which every row is its own
    segment: ``proj = x in_proj^T (+ bias)`` cut into (B | C | x), ``C * conv(B * x)`` with the
    rows' state slots read and shifted.  bfloat16, at most 64 rows, width a multiple of 16.
    Equals ``shortconv(linear(x, in_proj, in_bias), ...)``.  ``x`` may be ``ScaledRows`` or
    ``FragmentRows``."""
    scale = None
    if isinstance(x, ScaledRows):
        if (in_proj.dtype != BF16 or in_proj.dim() != 2 or in_proj.shape[1] != x.shape[1]
                or in_proj.data_ptr() % 16 or in_proj.shape[1] % 8):
            x = x.materialize()
        else:
            scale = x
            x = FragmentRows(x.data, x.shape[0], x.resid) if x.fragment else x.data
    a_frag, n_frag = 0, 0
    if isinstance(x, FragmentRows):
        if in_proj.dim() != 2 or in_proj.shape[1] != x.shape[1]:
            x = x.materialize()
        else:
            a_frag, n_frag, x = 1, x.shape[0], x.data
    _gpu("x", x, BF16, contiguous=False)
    _gpu_matrix("in_proj", in_proj, BF16)
    _gpu("taps", taps, F32)
    _gpu("state", state, F32)
    _gpu("seg_pos0", seg_pos0, I32)
    _gpu("seg_slot", seg_slot, I32)
    M, K = x.shape
    if a_frag:
        M = n_frag
    D, L = taps.shape
    _need(in_proj.shape == (3 * D, K), lambda: f"in_proj {tuple(in_proj.shape)} for D={D}, K={K}")
    _need(M <= 64 and D % 16 == 0, "linear_shortconv_step: at most 64 rows, width a multiple of 16")
    _need(seg_pos0.shape == (M,) and seg_slot.shape == (M,), "one segment a row")
    _need(L >= 2 and state.dim() == 3 and state.shape[1:] == (D, L - 1),
          lambda: f"state {tuple(state.shape)} for D={D}, L={L}")
    lda = x.stride(0) if M > 1 else K
    _need((x.stride(1) == 1 or K == 1) and K % 8 == 0 and lda % 8 == 0
          and x.data_ptr() % 16 == 0 and in_proj.data_ptr() % 16 == 0,
          "linear_shortconv_step: K and the row stride must be multiples of 8, tensors aligned")
    for n, t, shp in (("in_bias", in_bias, (3 * D,)), ("conv_bias", conv_bias, (D,))):
        if t is not None:
            _gpu(n, t, F32)
            _need(t.shape == shp, lambda: f"{n} must be {shp}")
    c_frag = _out_in_fragment_order(out_fragment, M, D, 0)
    out = torch.empty((16 if c_frag else M, D), dtype=BF16, device=x.device)
    check(library("gemm").kappai_gemm_bf16_shortconv_step(
        _ptr(x), *_matrix(in_proj, weight_frag), _ptr(in_bias), _ptr(out), _c_int(M),
        _c_int(D), _c_int(K),
        _c_int(lda), _ptr(taps), _ptr(conv_bias), _ptr(state), _ptr(seg_pos0), _ptr(seg_slot),
        _c_int(L), _c_int(a_frag), *(scale._scale_args() if scale is not None else _NO_SCALE),
        _c_int(1 if c_frag else 0), _stream()), "gemm_bf16_shortconv_step")
    return FragmentRows(out, M, None) if c_frag else out


# ---------------------------------------------------------------------------------------
def shortconv(proj: torch.Tensor, taps: torch.Tensor, bias: Optional[torch.Tensor],
              state: torch.Tensor, row_seg: torch.Tensor, seg_start: torch.Tensor,
              seg_pos0: torch.Tensor, seg_slot: torch.Tensor) -> torch.Tensor:
    """Gated causal depthwise convolution of ``proj`` [T, 3D] = (B | C | x) per segment with
    taps [D, L]; reads and then updates ``state`` [slots, D, L-1] (float32) of every
    segment's slot.  Returns C * conv(B * x) as [T, D].  ``proj`` may be the float32 partial
    sums [S, T, 3D] of a projection split over its input dimension: they are added in order and
    rounded to bfloat16 first, and the result is bfloat16."""
    _gpu("proj", proj, (F32, BF16))
    parts = None
    if proj.dim() == 3:
        _need(proj.dtype == F32, "shortconv: partial sums are float32")
        parts, proj = proj, proj[0]
    _gpu("taps", taps, F32)
    _gpu("state", state, F32)
    for n, t in (("row_seg", row_seg), ("seg_start", seg_start), ("seg_pos0", seg_pos0),
                 ("seg_slot", seg_slot)):
        _gpu(n, t, I32)
    T = proj.shape[0]
    D, L = taps.shape
    S = seg_pos0.shape[0]
    _need(proj.shape == (T, 3 * D), lambda: f"shortconv: proj {tuple(proj.shape)} for D={D}")
    _need(L >= 2 and state.dim() == 3 and state.shape[1:] == (D, L - 1),
          lambda: f"shortconv: state {tuple(state.shape)} for D={D}, L={L}")
    _need(row_seg.shape[0] == T and seg_start.shape[0] == S + 1 and seg_slot.shape[0] == S,
          "shortconv: segment tables do not fit the batch")
    _need(T <= 2 ** 31 - 1 and S >= 1, "shortconv: batch too large or empty")
    if bias is not None:
        _gpu("bias", bias, F32)
        _need(bias.shape == (D,), "shortconv: bias must be [D]")
    if parts is not None:
        out = torch.empty((T, D), dtype=BF16, device=proj.device)
        check(library("shortconv").kappai_shortconv_parts(
            _ptr(parts), _c_int(parts.shape[0]), _ptr(taps), _ptr(bias), _ptr(state), _ptr(out),
            _ptr(row_seg), _ptr(seg_start), _ptr(seg_pos0), _ptr(seg_slot), _c_int(T), _c_int(S),
            _c_int(D), _c_int(L), _stream()), "shortconv_parts")
        return out
    out = torch.empty((T, D), dtype=proj.dtype, device=proj.device)
    check(library("shortconv").kappai_shortconv(
        _ptr(proj), _ptr(taps), _ptr(bias), _ptr(state), _ptr(out), _ptr(row_seg), _ptr(seg_start),
        _ptr(seg_pos0), _ptr(seg_slot), _c_int(T), _c_int(S), _c_int(D), _c_int(L),
        _c_int(_is_bf16(proj.dtype)), _stream()), "shortconv")
    return out


ROT_NONE, ROT_HALF, ROT_INTERLEAVED = 0, 1, 2
ATTENTION_TILE_ROWS = 32      # rows of a segment that one wave of the prefill kernel takes


def _check_pools(k_pool, v_pool, G, page_size, d) -> None:
    _need(k_pool.dim() == 4 and v_pool.dim() == 4 and k_pool.shape[0] == v_pool.shape[0]
          and tuple(k_pool.shape[1:]) == (G, page_size, d)
          and tuple(v_pool.shape[1:]) == (G, d, page_size),
          lambda: f"pools {tuple(k_pool.shape)} / {tuple(v_pool.shape)} are not keys [pages, {G}, "
          f"{page_size}, {d}] and transposed values [pages, {G}, {d}, {page_size}]")


def qk_norm_rope_store(qkv: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int,
                       q_norm_w: Optional[torch.Tensor], k_norm_w: Optional[torch.Tensor],
                       eps: float, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
                       rot_dim: int, rot_mode: int, k_pool: Optional[torch.Tensor],
                       v_pool: Optional[torch.Tensor], row_pos: torch.Tensor,
                       row_seg: torch.Tensor, block_tables: torch.Tensor, page_size: int,
                       store_kv: bool = True) -> torch.Tensor:
    """In ``qkv`` [T, (H + 2G) d]: normalise every q and k head, rotate them at the row's
    position (tables [positions, rot_dim/2]), rewrite q in place and store k and v into the
    pools [pages, G, page_size, d] through the block tables [S, max_blocks].  Returns the
    tensor whose leading H d columns hold q: ``qkv`` itself, or, when ``qkv`` is the float32
    partial sums [S, T, width] of a projection split over its input dimension (they are added
    in order and rounded to bfloat16 first), a new bfloat16 [T, H d]."""
    H, G, d = n_heads, n_kv_heads, head_dim
    _gpu("qkv", qkv, (F32, BF16))
    width = (H + 2 * G) * d if store_kv else H * d
    parts = qkv if qkv.dim() == 3 else None
    if parts is not None:
        _need(parts.dtype == F32 and parts.shape[2] >= width and parts.is_contiguous(),
              lambda: f"qk_norm_rope_store: partial sums {tuple(parts.shape)}")
        T = parts.shape[1]
        q_out = torch.empty((T, H * d), dtype=BF16, device=parts.device)
        row_stride, data_dtype = parts.shape[2], BF16
    else:
        T = qkv.shape[0]
        _need(qkv.dim() == 2 and qkv.shape[1] >= width,
              lambda: f"qk_norm_rope_store: qkv {tuple(qkv.shape)}")
        q_out, row_stride, data_dtype = None, qkv.stride(0), qkv.dtype
    _need(1 <= d <= MAX_HEAD_DIM,
          lambda: f"head_dim {d} is beyond the kernels' limit {MAX_HEAD_DIM}")
    _need(H + 2 * G <= MAX_GRID_Y, "too many heads for one launch")
    for n, t in (("q_norm_w", q_norm_w), ("k_norm_w", k_norm_w)):
        if t is not None:
            _gpu(n, t, F32)
            _need(t.shape == (d,), lambda: f"{n} must be [head_dim]")
    if rot_mode != ROT_NONE:
        _gpu("cos", cos, F32)
        _gpu("sin", sin, F32)
        _need(rot_dim % 2 == 0 and 0 < rot_dim <= d, lambda: f"rot_dim {rot_dim} for head_dim {d}")
        _need(cos.shape == sin.shape and cos.dim() == 2 and cos.shape[1] == rot_dim // 2,
              "rotation tables must be [positions, rot_dim/2]")
    _gpu("row_pos", row_pos, I32)
    _gpu("row_seg", row_seg, I32)
    _need(row_pos.shape[0] == T and row_seg.shape[0] == T, "row tables do not fit the batch")
    max_blocks = 0
    if store_kv:
        _gpu("k_pool", k_pool, data_dtype)
        _gpu("v_pool", v_pool, data_dtype)
        _gpu("block_tables", block_tables, I32)
        _check_pools(k_pool, v_pool, G, page_size, d)
        _need(block_tables.dim() == 2, "block_tables must be [segments, max_blocks]")
        max_blocks = block_tables.shape[1]
    check(library("attention").kappai_qk_norm_rope_store(
        _ptr(None if parts is not None else qkv), _c_int(row_stride), _ptr(q_norm_w),
        _ptr(k_norm_w), _c_float(eps), _ptr(cos),
        _ptr(sin), _c_int(rot_dim if rot_mode else 0), _c_int(rot_mode), _ptr(k_pool),
        _ptr(v_pool), _ptr(row_pos), _ptr(row_seg), _ptr(block_tables if store_kv else None),
        _c_int(max_blocks), _c_int(T), _c_int(H), _c_int(G), _c_int(d), _c_int(page_size),
        _c_int(1 if store_kv else 0), _c_int(_is_bf16(data_dtype)), _ptr(parts),
        _c_int(parts.shape[0] if parts is not None else 0), _ptr(q_out),
        _c_int(H * d), _stream()), "qk_norm_rope_store")
    return qkv if parts is None else q_out


class ScoreModsC(ctypes.Structure):
    """``kappai_score_mods`` of csrc/score_mods.h."""
    _fields_ = [("softcap", _c_float), ("dist_bias", _vp), ("dist_cols", _c_int), ("sink", _vp)]


@dataclass(frozen=True)
class ScoreMods:
    """What the attention kernels do to a score between the scaled dot product and the softmax:
    ``softcap`` (0: nothing; else ``softcap * tanh(score / softcap)``); ``distance_bias`` float32
    [H, n], added after the cap, column ``min(i - j, n - 1)`` for query position i and key
    position j; ``sink`` float32 [H]: ``exp(sink[h])`` joins the softmax's denominator once, with
    no key and no value behind it."""
    softcap: float = 0.0
    distance_bias: Optional[torch.Tensor] = None
    sink: Optional[torch.Tensor] = None

    def active(self) -> bool:
        return self.softcap > 0.0 or self.distance_bias is not None or self.sink is not None

    def c_struct(self, n_heads: int) -> "ScoreModsC":
        cols = 0
        if self.distance_bias is not None:
            _gpu("distance_bias", self.distance_bias, F32)
            _need(self.distance_bias.dim() == 2 and self.distance_bias.shape[0] == n_heads
                  and self.distance_bias.shape[1] >= 1,
                  lambda: f"distance_bias {tuple(self.distance_bias.shape)} for {n_heads} heads")
            cols = self.distance_bias.shape[1]
        if self.sink is not None:
            _gpu("sink", self.sink, F32)
            _need(self.sink.shape == (n_heads,), lambda: f"sink {tuple(self.sink.shape)}")
        return ScoreModsC(float(self.softcap),
                          0 if self.distance_bias is None else self.distance_bias.data_ptr(), cols,
                          0 if self.sink is None else self.sink.data_ptr())


@dataclass
class QkPrologue:
    """What the decode attention kernels do themselves when they are given the projection as it
    comes out of its product: per-head RMSNorm of q and k (weights [d] float32, or None), the
    rotate-half rotation over the whole head (``cos`` / ``sin`` [positions, d / 2] float32, or
    None for no rotation), and with ``store_kv`` the storing of each row's own key and value
    (which then stand beside q in the projection: q heads, k heads, v heads)."""
    q_norm_w: Optional[torch.Tensor]
    k_norm_w: Optional[torch.Tensor]
    eps: float
    cos: Optional[torch.Tensor]
    sin: Optional[torch.Tensor]
    store_kv: bool = True


def keys_bound(max_position: int, window: int) -> int:
    """An upper bound of the keys a row at ``max_position`` or before sees (``window``: 0 all,
    n > 0 a sliding window of n, n < 0 chunks of -n positions; rounded as the kernels' tiles)."""
    return min(max_position + 1, abs(window)) + 32 if window else max_position + 1


def decode_form(n_heads: int, n_kv_heads: int, head_dim: int, max_position: int,
                window: int = 0) -> str:
    """Which of the two decode kernels a step takes: with few keys ("decode-block") a block per
    (row, kv head) splits them over its waves and merges in LDS; else ("decode-split") the keys
    are split over blocks, whose partial results a second kernel merges."""
    n_keys = keys_bound(max_position, window)
    lib = library("attention_mfma", HEAD_DIM=head_dim)
    block_waves = lib.kappai_attn_decode_block_waves(n_heads // n_kv_heads)
    return "decode-block" if block_waves and n_keys <= DECODE_BLOCK_MAX_KEYS else "decode-split"


def decode_takes_qk(head_dim: int, page_size: int) -> bool:
    """Whether the decode attention kernels of this head size take a ``QkPrologue`` (head sizes
    64 and 128: a lane holds both halves of a rotation pair, and the registers the prologue)."""
    if head_dim % 16 or head_dim > 256 or page_size % 16:
        return False
    return bool(library("attention_mfma", HEAD_DIM=head_dim).kappai_attn_decode_takes_qk())


def paged_attention(q: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int,
                    k_pool: torch.Tensor, v_pool: torch.Tensor, row_pos: torch.Tensor,
                    row_seg: torch.Tensor, block_tables: torch.Tensor, page_size: int,
                    scale: float, window: int = 0, q_tiles: Optional[torch.Tensor] = None,
                    single_rows: bool = False, max_position: Optional[int] = None,
                    kernel: str = "auto", prefill_variant: int = 0,
                    qk: Optional[QkPrologue] = None, lone_rows: Optional[torch.Tensor] = None,
                    max_lone_position: int = -1,
                    mods: Optional[ScoreMods] = None, chunk: int = 0) -> torch.Tensor:
    """Causal attention of every row over the keys of its request that are in the cache
    (its own included; the last ``window`` of them when a window is set; with ``chunk`` those of
    its own chunk of that many positions, chunks counted from position 0: the kernels take a
    chunk as a negative window).  ``q`` is
    [T, >= H d] with a row stride (the q columns of the fused projection).  Returns [T, H d].

    bfloat16 with a page size and head size that are multiples of 16 runs on the matrix
    cores: the split-key decode kernel when every segment is a single row (``single_rows``;
    ``max_position`` sizes the splits), else the tiled kernel over ``q_tiles`` [tiles, 4] =
    (segment, first row, rows <= 32, place of the tile in its segment: index | tiles << 16, or 0).
    Everything else, float32 included, runs the plain
    kernel.  ``kernel`` = "rows" | "prefill" | "decode" | "decode-block" | "decode-split" forces
    one (for tests);
    ``prefill_variant`` 1 / 2 forces the tiled kernel's form (2: key tiles shared by four query
    heads of a kv head through LDS; head sizes 64 and 128 only).

    ``qk`` (decode kernels only, see ``decode_takes_qk``): ``q`` is the raw projection and the
    kernel normalises and rotates q and the rows' own keys itself and stores keys and values.

    ``lone_rows`` (int32, with ``max_lone_position``; tiled kernel only): rows that ``q_tiles``
    leaves out, the single decoded tokens of a step that also holds prompt portions.  They go
    through the decode kernel that splits keys over blocks.

    ``mods`` (``ScoreMods``): a cap on the scores, a bias by distance, a sink."""
    H, G, d = n_heads, n_kv_heads, head_dim
    _need(not (window and chunk) and (window or 0) >= 0 and chunk >= 0,
          "paged_attention: a sliding window or chunks, not both")
    if chunk:
        # (while no position of the step has left the first chunk, a chunk is the whole past:
        # the kernels' plain form, which pairs the tiles of a portion for equal work)
        first_chunk_only = max_position is not None and 0 <= max_position < chunk
        window = 0 if first_chunk_only else -int(chunk)
    if mods is not None and not mods.active():
        mods = None
    mods_c = mods.c_struct(H) if mods is not None else None
    mods_ref = ctypes.byref(mods_c) if mods_c is not None else None
    _gpu("q", q, (F32, BF16), contiguous=False)
    T = q.shape[0]
    _need(q.dim() == 2 and q.shape[1] >= H * d and (q.stride(1) == 1),
          lambda: f"paged_attention: q {tuple(q.shape)}")
    _need(d % 8 == 0 and d <= MAX_HEAD_DIM,
          lambda: f"head_dim {d}: the attention kernels take multiples of 8 up to {MAX_HEAD_DIM}")
    _need(G >= 1 and H % G == 0 and H <= MAX_GRID_Y, lambda: f"{H} heads over {G} kv heads")
    _gpu("k_pool", k_pool, q.dtype)
    _gpu("v_pool", v_pool, q.dtype)
    _check_pools(k_pool, v_pool, G, page_size, d)
    _gpu("row_pos", row_pos, I32)
    _gpu("row_seg", row_seg, I32)
    _gpu("block_tables", block_tables, I32)
    _need(row_pos.shape[0] == T and row_seg.shape[0] == T and block_tables.dim() == 2,
          "row tables do not fit the batch")
    out = torch.empty((T, H * d), dtype=q.dtype, device=q.device)
    mfma_ok = (q.dtype == BF16 and page_size % 16 == 0 and d % 16 == 0 and d <= 256
               and q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0)
    if kernel == "auto":
        if not mfma_ok:
            kernel = "rows"
        elif single_rows and H // G <= 16 and max_position is not None:
            kernel = "decode"
        elif q_tiles is not None:
            kernel = "prefill"
        else:
            kernel = "rows"
    if kernel == "rows":
        check(library("attention").kappai_paged_attention_rows_scored(
            _ptr(q), _c_int(q.stride(0)), _ptr(k_pool), _ptr(v_pool), _ptr(out), _c_int(H * d),
            _ptr(row_pos), _ptr(row_seg), _ptr(block_tables), _c_int(block_tables.shape[1]),
            _c_int(T), _c_int(H), _c_int(G), _c_int(d), _c_int(page_size), _c_int(window or 0),
            _c_float(scale), _c_int(_is_bf16(q.dtype)), mods_ref, _stream()),
            "paged_attention_rows")
        return out
    _need(mfma_ok, "the matrix-core attention kernels need bfloat16, a page size and a head size "
          f"that are multiples of 16 (head size at most 256) and 16-byte aligned rows; got "
          f"{q.dtype}, page {page_size}, head {d}")
    lib = library("attention_mfma", HEAD_DIM=d)
    if kernel == "prefill":
        _gpu("q_tiles", q_tiles, I32)
        _need(q_tiles.dim() == 2 and q_tiles.shape[1] == 4, "q_tiles must be [tiles, 4]")
        check(lib.kappai_attn_prefill_scored(
            _ptr(q), _c_int(q.stride(0)), _ptr(k_pool), _ptr(v_pool), _ptr(out), _c_int(H * d),
            _ptr(q_tiles), _c_int(q_tiles.shape[0]), _ptr(row_pos), _ptr(block_tables),
            _c_int(block_tables.shape[1]), _c_int(H), _c_int(G), _c_int(page_size),
            _c_int(window or 0), _c_float(scale), _c_int(prefill_variant), mods_ref, _stream()),
            "attn_prefill")
        if lone_rows is not None:
            _gpu("lone_rows", lone_rows, I32)
            _need(H // G <= 16 and lone_rows.dim() == 1 and max_lone_position >= 0,
                  "paged_attention: rows left out of the tiles need the decode kernel (at most 16 "
                  "query heads a kv head) and their largest position")
            _decode_split(lib, q, H, G, d, k_pool, v_pool, row_pos, row_seg, block_tables,
                          page_size, scale, window, max_lone_position, out, lone_rows,
                          mods_ref=mods_ref)
        return out
    _need(kernel in ("decode", "decode-block", "decode-split"),
          lambda: f"unknown attention kernel {kernel!r}")
    _need(H // G <= 16, "the decode kernel takes at most 16 query heads per kv head")
    _need(max_position is not None, "the decode kernel needs the batch's largest position")
    qk_args = ()
    _need(qk is None or mods is None, "paged_attention: the decode kernels do either the norm and "
          "the rotation themselves or work on the scores, not both")
    if qk is not None:
        _need(bool(lib.kappai_attn_decode_takes_qk()),
              lambda: f"the decode kernels of head size {d} do not take the norm and the rotation")
        _need(q.shape[1] >= (H + 2 * G) * d if qk.store_kv else True,
              "paged_attention: keys and values to store must stand beside q in the projection")
        for name, w in (("q_norm_w", qk.q_norm_w), ("k_norm_w", qk.k_norm_w)):
            if w is not None:
                _gpu(name, w, F32)
                _need(w.shape == (d,), lambda: f"{name}: one weight for each of the {d} of a head")
        _need((qk.cos is None) == (qk.sin is None), "cos and sin tables come together")
        if qk.cos is not None:
            _gpu("cos", qk.cos, F32)
            _gpu("sin", qk.sin, F32)
            _need(qk.cos.shape == qk.sin.shape and qk.cos.dim() == 2
                  and qk.cos.shape[1] == d // 2 and qk.cos.shape[0] > max_position,
                  lambda: f"rotation tables {tuple(qk.cos.shape)} for positions up to "
                          f"{max_position} of heads of {d}")
        qk_args = (_ptr(qk.q_norm_w), _ptr(qk.k_norm_w), _c_float(qk.eps), _ptr(qk.cos),
                   _ptr(qk.sin), _c_int(1 if qk.store_kv else 0))
    n_keys = keys_bound(max_position, window)
    block_waves = lib.kappai_attn_decode_block_waves(H // G)
    if kernel == "decode":
        kernel = "decode-split" if qk is not None else decode_form(H, G, d, max_position, window)
    if kernel == "decode-block":
        _need(block_waves > 0, "too many query heads a kv head for the block form")
        _need(qk is None, "the decode kernel that keeps a row's keys in one block takes q ready "
                          "made and the keys stored")
        check(lib.kappai_attn_decode_block_scored(
            _ptr(q), _c_int(q.stride(0)), _ptr(k_pool), _ptr(v_pool), _ptr(out), _c_int(H * d),
            _ptr(row_pos), _ptr(row_seg), _ptr(block_tables), _c_int(block_tables.shape[1]),
            _c_int(T), _c_int(H), _c_int(G), _c_int(page_size), _c_int(window or 0),
            _c_float(scale), _c_int(block_waves), mods_ref, _stream()), "attn_decode_block")
        return out
    _decode_split(lib, q, H, G, d, k_pool, v_pool, row_pos, row_seg, block_tables, page_size, scale,
                  window, max_position, out, None, qk_args, mods_ref=mods_ref)
    return out


def decode_splits(keys_per_wave: int, rows: int, n_kv_heads: int, n_keys: int):
    """(fewest keys a split, most splits a row) of the decode kernel that splits keys over blocks:
    the rule lives in C (``kappai_decode_splits``), where a step launched from C uses it too."""
    kps, n = _c_int(0), _c_int(0)
    library("engine").kappai_decode_splits(
        _c_int(keys_per_wave), _c_int(DECODE_MAX_SPLITS), _c_int(DECODE_WAVES), _c_int(rows),
        _c_int(n_kv_heads), _c_int(n_keys), ctypes.byref(kps), ctypes.byref(n))
    return kps.value, n.value


def _decode_split(lib, q, H, G, d, k_pool, v_pool, row_pos, row_seg, block_tables, page_size, scale,
                  window, max_position, out, row_ids, qk_args=(), mods_ref=None):
    """The decode kernel that splits a row's keys over blocks, and its merge, for all rows or
    (``row_ids``) some of them."""
    T = q.shape[0] if row_ids is None else row_ids.shape[0]
    n_keys = keys_bound(max_position, window)
    # one wave keeps the loads of `kpw` keys in flight; splits are whole numbers of that, and
    # at most DECODE_MAX_SPLITS of them are merged
    kpw = lib.kappai_attn_keys_per_wave()
    # and no more splits than DECODE_WAVES blocks: with many rows a wave rather takes several
    # chunks in turn than writes a partial result for each.  These are the most splits and the
    # fewest keys a split of this step; the kernels settle on a number of keys a split from the
    # rows' own lengths (step_keys_per_split in csrc/attention_mfma.hip) and leave the rest of
    # the splits empty.
    keys_per_split, n_splits = decode_splits(kpw, T, G, n_keys)
    part_o = torch.empty((T, H, n_splits, d), dtype=F32, device=q.device)
    part_ml = torch.empty((T, H, n_splits, 2), dtype=F32, device=q.device)
    head = (_ptr(q), _c_int(q.stride(0)), _ptr(k_pool), _ptr(v_pool), _ptr(out), _c_int(H * d),
            _ptr(part_o), _ptr(part_ml))
    tail = (_ptr(row_pos), _ptr(row_seg), _ptr(block_tables), _c_int(block_tables.shape[1]),
            _c_int(T), _c_int(H), _c_int(G), _c_int(page_size), _c_int(window or 0),
            _c_float(scale), _c_int(keys_per_split), _c_int(n_splits))
    if mods_ref is not None:
        check(lib.kappai_attn_decode_scored(*head, _ptr(row_ids), *tail, mods_ref, _stream()),
              "attn_decode_scored")
    elif row_ids is not None:
        check(lib.kappai_attn_decode_rows(*head, _ptr(row_ids), *tail, _stream()),
              "attn_decode_rows")
    elif qk_args:
        check(lib.kappai_attn_decode_qk(*head, *tail, *qk_args, _stream()), "attn_decode_qk")
    else:
        check(lib.kappai_attn_decode(*head, *tail, _stream()), "attn_decode")


# ---------------------------------------------------------------------------------------
def _also(also: Optional[torch.Tensor], n: int) -> _vp:
    if also is None:
        return _vp(0)
    _gpu("also", also, I32)
    _need(also.shape == (n,), "also: a second place for one token a row")
    return _vp(also.data_ptr())


def sample_rows(logits: torch.Tensor, temperature: torch.Tensor, uniform: torch.Tensor,
                out: Optional[torch.Tensor] = None,
                also: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token per row of ``logits`` [n, V] (float32): argmax (lowest id on ties) where the
    row's temperature is <= 0, else an inverse-CDF draw of softmax(logits / T) at the row's
    uniform number.  ``out`` (int32 [n]) receives the tokens when given, ``also`` (int32 [n])
    receives them as well (the token table of the step that comes next)."""
    _gpu("logits", logits, F32)
    _gpu("temperature", temperature, F32)
    _gpu("uniform", uniform, F32)
    n, V = logits.shape
    _need(temperature.shape == (n,) and uniform.shape == (n,), "one temperature and uniform a row")
    if out is None:
        out = torch.empty((n,), dtype=I32, device=logits.device)
    else:
        _gpu("out", out, I32)
        _need(out.shape == (n,), "sample_rows: out must hold one token a row")
    check(library("sampling").kappai_sample_rows(
        _ptr(logits), _ptr(temperature), _ptr(uniform), _ptr(out), _also(also, n), _c_int(n),
        _c_int(V), _stream()), "sample_rows")
    return out


FILTER_MAX_KEEP = 1024     # candidates the filtered-sampling kernel can hold


def sample_filtered(logits: torch.Tensor, rows: torch.Tensor, keep: torch.Tensor,
                    temperature: torch.Tensor, top_p: torch.Tensor, min_p: torch.Tensor,
                    uniform: torch.Tensor, out: torch.Tensor, wide: bool = False,
                    also: Optional[torch.Tensor] = None) -> None:
    """For every entry i: draw a token for row ``rows[i]`` of ``logits`` from its ``keep[i]``
    largest logits after temperature, top-p and min-p, at ``uniform[i]``, and write it to
    ``out[rows[i]]`` (int32).  ``keep[i]`` is at most ``FILTER_MAX_KEEP``, or, with ``wide``, any
    number up to the vocabulary (a slower kernel that sorts whole rows in a workspace).  ``also``:
    a second tensor like ``out`` that receives the same tokens."""
    _gpu("logits", logits, F32)
    _gpu("rows", rows, I32)
    _gpu("keep", keep, I32)
    _gpu("out", out, I32)
    n = rows.shape[0]
    for name, t in (("temperature", temperature), ("top_p", top_p), ("min_p", min_p),
                    ("uniform", uniform)):
        _gpu(name, t, F32)
        _need(t.shape == (n,), lambda: f"{name}: one value per entry")
    _need(keep.shape == (n,) and out.shape == (logits.shape[0],), "sample_filtered: table sizes")
    if wide:
        lib = library("sampling")
        n2 = int(lib.kappai_sample_filtered_wide_n2(_c_int(logits.shape[1])))
        ws_val = torch.empty((n, n2), dtype=F32, device=logits.device)
        ws_idx = torch.empty((n, n2), dtype=I32, device=logits.device)
        check(lib.kappai_sample_filtered_wide(
            _ptr(logits), _ptr(rows), _ptr(keep), _ptr(temperature), _ptr(top_p), _ptr(min_p),
            _ptr(uniform), _ptr(out), _also(also, logits.shape[0]), _c_int(n),
            _c_int(logits.shape[1]), _ptr(ws_val), _ptr(ws_idx), _stream()), "sample_filtered_wide")
        return
    check(library("sampling").kappai_sample_filtered(
        _ptr(logits), _ptr(rows), _ptr(keep), _ptr(temperature), _ptr(top_p), _ptr(min_p),
        _ptr(uniform), _ptr(out), _also(also, logits.shape[0]), _c_int(n), _c_int(logits.shape[1]),
        _stream()), "sample_filtered")


def repeat_penalty(logits: torch.Tensor, row_start: torch.Tensor, tokens: torch.Tensor,
                   penalty: torch.Tensor) -> None:
    """In place: for row r and each token in ``tokens[row_start[r]:row_start[r+1]]`` divide a
    positive logit by ``penalty[r]`` and multiply any other by it."""
    _gpu("logits", logits, F32)
    _gpu("row_start", row_start, I32)
    _gpu("tokens", tokens, I32)
    _gpu("penalty", penalty, F32)
    n, V = logits.shape
    _need(row_start.shape == (n + 1,) and penalty.shape == (n,), "repeat_penalty: tables per row")
    check(library("sampling").kappai_repeat_penalty(
        _ptr(logits), _ptr(row_start), _ptr(tokens), _ptr(penalty), _c_int(n), _c_int(V),
        _stream()), "repeat_penalty")


def history_set(history: torch.Tensor, seen: torch.Tensor, slots: torch.Tensor,
                starts: torch.Tensor, tokens: torch.Tensor) -> None:
    """``history[slots[i]]`` (a ring of token ids, int32 [slots, cap]) becomes
    ``tokens[starts[i]:starts[i+1]]`` (at most cap, the oldest first) and ``seen[slots[i]]`` their
    number: what a request has seen before its first token is chosen on the GPU."""
    for name, t in (("history", history), ("seen", seen), ("slots", slots), ("starts", starts),
                    ("tokens", tokens)):
        _gpu(name, t, I32)
    n = slots.shape[0]
    _need(history.dim() == 2 and seen.shape == (history.shape[0],) and starts.shape == (n + 1,),
          "history_set: a ring and a count per slot, starts per entry")
    check(library("sampling").kappai_history_set(
        _ptr(history), _ptr(seen), _ptr(slots), _ptr(starts), _ptr(tokens), _c_int(n),
        _c_int(history.shape[1]), _stream()), "history_set")


def repeat_penalty_history(logits: torch.Tensor, rows: torch.Tensor, slots: torch.Tensor,
                           penalty: torch.Tensor, last_n: torch.Tensor, history: torch.Tensor,
                           seen: torch.Tensor) -> None:
    """In place: for entry i the repeat penalty ``penalty[i]`` of row ``rows[i]`` over the last
    ``last_n[i]`` tokens of ``history[slots[i]]``, once per occurrence as ``repeat_penalty``
    applies it to a list."""
    _gpu("logits", logits, F32)
    _gpu("penalty", penalty, F32)
    for name, t in (("rows", rows), ("slots", slots), ("last_n", last_n), ("history", history),
                    ("seen", seen)):
        _gpu(name, t, I32)
    n = rows.shape[0]
    _need(slots.shape == (n,) and penalty.shape == (n,) and last_n.shape == (n,)
          and history.dim() == 2 and seen.shape == (history.shape[0],),
          "repeat_penalty_history: tables per entry, a ring and a count per slot")
    check(library("sampling").kappai_repeat_penalty_history(
        _ptr(logits), _ptr(rows), _ptr(slots), _ptr(penalty), _ptr(last_n), _ptr(history),
        _ptr(seen), _c_int(n), _c_int(logits.shape[1]), _c_int(history.shape[1]), _stream()),
        "repeat_penalty_history")


def history_append(chosen: torch.Tensor, rows: torch.Tensor, slots: torch.Tensor,
                   history: torch.Tensor, seen: torch.Tensor) -> None:
    """The token ``chosen[rows[i]]`` joins ``history[slots[i]]`` for every entry i."""
    for name, t in (("chosen", chosen), ("rows", rows), ("slots", slots), ("history", history),
                    ("seen", seen)):
        _gpu(name, t, I32)
    n = rows.shape[0]
    _need(slots.shape == (n,) and history.dim() == 2 and seen.shape == (history.shape[0],),
          "history_append: tables per entry, a ring and a count per slot")
    check(library("sampling").kappai_history_append(
        _ptr(chosen), _ptr(rows), _ptr(slots), _ptr(history), _ptr(seen), _c_int(n),
        _c_int(history.shape[1]), _stream()), "history_append")


# ---------------------------------------------------------------------------------------
# grouped RMS norm, the input convolution of a sublayer, scaled embedding with positions
# ---------------------------------------------------------------------------------------
def add_group_rmsnorm(resid: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor,
                      eps: float, groups: int, out_dtype, rows: Optional[torch.Tensor] = None,
                      write_resid: bool = True) -> torch.Tensor:
    """``resid += delta`` in float32 (``delta``: [T, D] bfloat16 or float32, float32 partial sums
    [S, T, D] added in order, or None), then every one of ``groups`` equal consecutive parts of a
    row divided by ``sqrt(mean(part^2) + eps)`` and the row multiplied by ``weight``.  With
    ``rows`` only those rows are summed and normalised and the residual is left alone.  Returns
    [n, D] in ``out_dtype``."""
    _gpu("resid", resid, F32)
    _gpu("weight", weight, F32)
    T, D = resid.shape
    _need(weight.shape == (D,) and groups >= 1 and D % groups == 0,
          lambda: f"add_group_rmsnorm: a width of {D} in {groups} groups, weight "
                  f"{tuple(weight.shape)}")
    _need((D + groups) * 4 <= 64 * 1024, lambda: f"add_group_rmsnorm: a width of {D} is beyond "
          "what the kernel keeps of a row")
    kind, n_part = 0, 0
    if delta is not None:
        _gpu("delta", delta, (F32, BF16))
        if delta.dim() == 3:
            _need(delta.dtype == F32 and tuple(delta.shape[1:]) == (T, D),
                  lambda: f"add_group_rmsnorm: partial sums {tuple(delta.shape)}")
            kind, n_part = 2, delta.shape[0]
        else:
            _need(tuple(delta.shape) == (T, D), lambda: f"add_group_rmsnorm: delta "
                  f"{tuple(delta.shape)} for a residual {tuple(resid.shape)}")
            kind, n_part = (1, 0) if delta.dtype == BF16 else (2, 1)
    n = T
    if rows is not None:
        _gpu("rows", rows, I32)
        n = rows.shape[0]
    out = torch.empty((n, D), dtype=out_dtype, device=resid.device)
    check(library("groupnorm").kappai_add_group_rmsnorm(
        _ptr(resid), _ptr(delta), _c_int(kind), _c_int(n_part), _c_int(T), _c_int(D),
        _ptr(weight), _c_float(eps), _c_int(groups), _ptr(rows), _c_int(n), _ptr(out),
        _c_int(_is_bf16(out_dtype)), _c_int(1 if write_resid and rows is None else 0),
        _stream()), "add_group_rmsnorm")
    return out


CANON_MAX_TAPS = 16


def canon_conv(h: torch.Tensor, taps: torch.Tensor, state: torch.Tensor, row_pos: torch.Tensor,
               row_seg: torch.Tensor, seg_start: torch.Tensor, seg_slot: torch.Tensor,
               out_dtype) -> torch.Tensor:
    """``h + conv(h)`` for float32 rows ``h`` [T, D]: ``conv(h)[t] = sum_j taps[:, j] *
    h[t - n + 1 + j]`` along each request's sequence, inputs before the step's rows taken from
    ``state`` [slots, n - 1, D] (the request's last n - 1 inputs, oldest first), zeros before
    position 0.  The state is brought up to date.  Returns [T, D] in ``out_dtype``."""
    _gpu("h", h, F32)
    _gpu("taps", taps, F32)
    _gpu("state", state, F32)
    T, D = h.shape
    n = taps.shape[1]
    _need(taps.shape[0] == D and 1 <= n <= CANON_MAX_TAPS,
          lambda: f"canon_conv: taps {tuple(taps.shape)} for a width of {D} (at most "
                  f"{CANON_MAX_TAPS} taps)")
    _need(state.dim() == 3 and tuple(state.shape[1:]) == (max(n - 1, 0), D),
          lambda: f"canon_conv: state {tuple(state.shape)} is not [slots, {n - 1}, {D}]")
    for name, t in (("row_pos", row_pos), ("row_seg", row_seg), ("seg_start", seg_start),
                    ("seg_slot", seg_slot)):
        _gpu(name, t, I32)
    S = seg_slot.shape[0]
    _need(row_pos.shape[0] == T and row_seg.shape[0] == T and seg_start.shape[0] == S + 1,
          "canon_conv: row tables do not fit the batch")
    out = torch.empty((T, D), dtype=out_dtype, device=h.device)
    check(library("groupnorm").kappai_canon_conv(
        _ptr(h), _ptr(taps), _ptr(state), _ptr(row_pos), _ptr(row_seg), _ptr(seg_start),
        _ptr(seg_slot), _c_int(T), _c_int(S), _c_int(D), _c_int(n), _ptr(out),
        _c_int(_is_bf16(out_dtype)), _stream()), "canon_conv")
    return out


def add_group_rmsnorm_canon_step(resid: torch.Tensor, delta: Optional[torch.Tensor],
                                 weight: torch.Tensor, eps: float, groups: int,
                                 taps: torch.Tensor, state: torch.Tensor, row_pos: torch.Tensor,
                                 seg_slot: torch.Tensor, out_dtype) -> torch.Tensor:
    """``add_group_rmsnorm`` and ``canon_conv`` in one kernel for a step whose every segment is a
    single row (row t is segment t): the residual gets the sum, the state its shift."""
    _gpu("resid", resid, F32)
    _gpu("weight", weight, F32)
    _gpu("taps", taps, F32)
    _gpu("state", state, F32)
    _gpu("row_pos", row_pos, I32)
    _gpu("seg_slot", seg_slot, I32)
    T, D = resid.shape
    n = taps.shape[1]
    _need(weight.shape == (D,) and groups >= 1 and D % groups == 0 and (D + groups) * 4 <= 65536,
          lambda: f"add_group_rmsnorm_canon_step: a width of {D} in {groups} groups")
    _need(taps.shape[0] == D and 1 <= n <= CANON_MAX_TAPS and state.dim() == 3
          and tuple(state.shape[1:]) == (n - 1, D),
          lambda: f"add_group_rmsnorm_canon_step: taps {tuple(taps.shape)}, state "
                  f"{tuple(state.shape)}")
    _need(row_pos.shape[0] == T and seg_slot.shape[0] == T,
          "add_group_rmsnorm_canon_step: one row a segment is needed")
    kind, n_part = 0, 0
    if delta is not None:
        _gpu("delta", delta, (F32, BF16))
        if delta.dim() == 3:
            _need(delta.dtype == F32 and tuple(delta.shape[1:]) == (T, D),
                  lambda: f"add_group_rmsnorm_canon_step: partial sums {tuple(delta.shape)}")
            kind, n_part = 2, delta.shape[0]
        else:
            _need(tuple(delta.shape) == (T, D), "add_group_rmsnorm_canon_step: delta's shape")
            kind, n_part = (1, 0) if delta.dtype == BF16 else (2, 1)
    out = torch.empty((T, D), dtype=out_dtype, device=resid.device)
    check(library("groupnorm").kappai_add_group_rmsnorm_canon_step(
        _ptr(resid), _ptr(delta), _c_int(kind), _c_int(n_part), _c_int(T), _c_int(D),
        _ptr(weight), _c_float(eps), _c_int(groups), _ptr(taps), _ptr(state), _ptr(row_pos),
        _ptr(seg_slot), _c_int(n), _ptr(out), _c_int(_is_bf16(out_dtype)), _stream()),
        "add_group_rmsnorm_canon_step")
    return out


def scale_add_positions(x: torch.Tensor, scale: float, table: torch.Tensor,
                        row_pos: torch.Tensor) -> None:
    """``x[t] = x[t] * scale + table[row_pos[t]]`` in place on float32 rows.  The caller keeps
    positions inside the table; the kernel reads no row outside it whatever ``row_pos`` holds."""
    _gpu("x", x, F32)
    _gpu("table", table, (F32, BF16))
    _gpu("row_pos", row_pos, I32)
    T, D = x.shape
    _need(table.dim() == 2 and table.shape[1] == D and row_pos.shape[0] == T,
          lambda: f"scale_add_positions: x {tuple(x.shape)}, table {tuple(table.shape)}")
    check(library("groupnorm").kappai_scale_add_positions(
        _ptr(x), _c_float(scale), _ptr(table), _c_int(_is_bf16(table.dtype)), _ptr(row_pos),
        _c_int(T), _c_int(D), _c_int(table.shape[0]), _stream()), "scale_add_positions")


GLU_SILU, GLU_GELU_TANH = 0, 1


def glu(gate_up: torch.Tensor, kind: int) -> torch.Tensor:
    """``act(gate_up[:, :F]) * gate_up[:, F:]`` for a fused [T, 2F] projection; ``kind``:
    ``GLU_SILU`` or ``GLU_GELU_TANH`` (0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))))."""
    _gpu("gate_up", gate_up, (F32, BF16))
    _need(gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0, "glu: [T, 2F] is needed")
    _need(kind in (GLU_SILU, GLU_GELU_TANH), lambda: f"glu: unknown activation {kind}")
    T, F = gate_up.shape[0], gate_up.shape[1] // 2
    out = torch.empty((T, F), dtype=gate_up.dtype, device=gate_up.device)
    check(library("elementwise").kappai_glu(
        _ptr(gate_up), _ptr(out), _c_int(T), _c_int(F), _c_int(_is_bf16(gate_up.dtype)),
        _c_int(kind), _stream()), "glu")
    return out


# ---------------------------------------------------------------------------------------
# minGRU
# ---------------------------------------------------------------------------------------
def mingru_scan(proj: torch.Tensor, state: torch.Tensor, seg_start: torch.Tensor,
                seg_pos0: torch.Tensor, seg_slot: torch.Tensor, out_dtype,
                chunks: Optional[torch.Tensor] = None,
                seg_chunk0: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The minGRU recurrence over projections [T, 3W] = (update gate | candidate | output gate,
    biases added; float32, or bfloat16 when the output is bfloat16 too): ``S = (1 - z) S + z c`` with ``z = sigmoid``, ``c = u + 1/2`` for
    ``u >= 0`` and ``sigmoid(u)`` below, output ``S * silu(g)`` [T, W] in ``out_dtype``.  ``state``
    [slots, W] float32 is read (unless the segment starts at position 0) and left at the
    segment's last row.  ``chunks`` [n, 3] = (segment, first row, rows) with ``seg_chunk0`` [S + 1]:
    long segments are scanned chunk by chunk in three passes."""
    _gpu("proj", proj, (F32, BF16))
    _gpu("state", state, F32)
    T = proj.shape[0]
    _need(proj.dim() == 2 and proj.shape[1] % 3 == 0, lambda: f"mingru_scan: {tuple(proj.shape)}")
    _need(proj.dtype == F32 or out_dtype == BF16,
          "mingru_scan: bfloat16 projections give bfloat16 outputs")
    W = proj.shape[1] // 3
    _need(state.dim() == 2 and state.shape[1] == W,
          lambda: f"mingru_scan: state {tuple(state.shape)} for a width of {W}")
    for name, t in (("seg_start", seg_start), ("seg_pos0", seg_pos0), ("seg_slot", seg_slot)):
        _gpu(name, t, I32)
    S = seg_slot.shape[0]
    _need(seg_start.shape[0] == S + 1 and seg_pos0.shape[0] == S,
          "mingru_scan: segment tables do not fit")
    out = torch.empty((T, W), dtype=out_dtype, device=proj.device)
    n_chunks, carry = 0, None
    if chunks is not None:
        _gpu("chunks", chunks, I32)
        _gpu("seg_chunk0", seg_chunk0, I32)
        _need(chunks.dim() == 2 and chunks.shape[1] == 3 and seg_chunk0.shape[0] == S + 1,
              "mingru_scan: chunk tables do not fit")
        n_chunks = chunks.shape[0]
        carry = torch.empty((n_chunks, 3, W), dtype=F32, device=proj.device)
    check(library("mingru").kappai_mingru_scan(
        _ptr(proj), _c_int(_is_bf16(proj.dtype)), _ptr(state), _ptr(seg_start), _ptr(seg_pos0),
        _ptr(seg_slot), _c_int(T),
        _c_int(S), _c_int(W), _ptr(chunks), _ptr(seg_chunk0), _c_int(n_chunks), _ptr(carry),
        _ptr(out), _c_int(_is_bf16(out_dtype)), _stream()), "mingru_scan")
    return out


def gated_unit_scan(gates: torch.Tensor, gate_bias: torch.Tensor, u: torch.Tensor,
                    y: torch.Tensor, softplus_lam: torch.Tensor,
                    rate: float, state: torch.Tensor, seg_start: torch.Tensor,
                    seg_pos0: torch.Tensor, seg_slot: torch.Tensor,
                    chunks: Optional[torch.Tensor] = None,
                    seg_chunk0: Optional[torch.Tensor] = None, gate_part: int = 0) -> torch.Tensor:
    """The real-gated linear unit per channel: ``a = exp(-rate * sigmoid(g_r) * softplus_lam)``,
    ``S = a S + sqrt(1 - a^2) * sigmoid(g_i) * u``, output ``S * gelu_tanh(y)``.  ``gates``
    [T, 2W] float32 = (g_r | g_i) before the sigmoid and without ``gate_bias`` [2W], ``u`` [T, W], ``y`` [T, >= W] (a view with a
    row stride) as a product stored them, ``softplus_lam`` [W] float32, ``state`` [slots, W]
    float32.  ``gate_part`` > 0: ``gates`` and ``gate_bias`` are laid out block by block, (g_r | g_i)
    of ``gate_part`` channels each (what one product a block leaves), not (g_r | g_i) of all
    channels.  ``chunks`` / ``seg_chunk0`` as for ``mingru_scan``.  Returns [T, W] as ``u`` is
    stored."""
    _gpu("gates", gates, F32)
    _gpu("gate_bias", gate_bias, F32)
    _gpu("u", u, (F32, BF16))
    _gpu("y", y, u.dtype, contiguous=False)
    _gpu("softplus_lam", softplus_lam, F32)
    _gpu("state", state, F32)
    T, W = u.shape
    _need(tuple(gates.shape) == (T, 2 * W) and gate_bias.shape == (2 * W,) and y.dim() == 2 and y.shape[0] == T
          and y.shape[1] >= W and y.stride(1) == 1 and softplus_lam.shape == (W,)
          and state.dim() == 2 and state.shape[1] == W
          and gate_part >= 0 and (gate_part == 0 or W % gate_part == 0),
          lambda: f"gated_unit_scan: gates {tuple(gates.shape)}, u {tuple(u.shape)}, y "
                  f"{tuple(y.shape)}, state {tuple(state.shape)}")
    for name, t in (("seg_start", seg_start), ("seg_pos0", seg_pos0), ("seg_slot", seg_slot)):
        _gpu(name, t, I32)
    S = seg_slot.shape[0]
    _need(seg_start.shape[0] == S + 1 and seg_pos0.shape[0] == S,
          "gated_unit_scan: segment tables do not fit")
    out = torch.empty((T, W), dtype=u.dtype, device=u.device)
    n_chunks, carry = 0, None
    if chunks is not None:
        _gpu("chunks", chunks, I32)
        _gpu("seg_chunk0", seg_chunk0, I32)
        _need(chunks.dim() == 2 and chunks.shape[1] == 3 and seg_chunk0.shape[0] == S + 1,
              "gated_unit_scan: chunk tables do not fit")
        n_chunks = chunks.shape[0]
        carry = torch.empty((n_chunks, 3, W), dtype=F32, device=u.device)
    check(library("mingru").kappai_gated_unit_scan(
        _ptr(gates), _ptr(gate_bias), _ptr(u), _ptr(y), _c_int(y.stride(0)), _ptr(softplus_lam),
        _c_float(rate), _c_int(gate_part),
        _c_int(_is_bf16(u.dtype)), _ptr(state), _ptr(seg_start), _ptr(seg_pos0), _ptr(seg_slot),
        _c_int(T), _c_int(S), _c_int(W), _ptr(chunks), _ptr(seg_chunk0), _c_int(n_chunks),
        _ptr(carry), _ptr(out), _stream()), "gated_unit_scan")
    return out


GATED_UNIT_STEP_MAX_PART = 4096     # channels a block that the one-kernel decode step takes


def gated_unit_step(proj: torch.Tensor, taps: torch.Tensor, conv_bias: torch.Tensor,
                    conv_state: torch.Tensor, gate_w: torch.Tensor, gate_bias: torch.Tensor,
                    softplus_lam: torch.Tensor, rate: float, state: torch.Tensor,
                    seg_pos0: torch.Tensor, seg_slot: torch.Tensor) -> torch.Tensor:
    """A step of single rows (row t is segment t) through the real-gated unit in one kernel:
    ``conv_silu`` without activation, both gates of every block, ``gated_unit_scan`` and the
    states brought up to date.  ``proj`` [T, >= 2W] = (x | y) with biases added (a view with a
    row stride), ``taps`` [W, n] float32, ``conv_bias`` [W], ``conv_state`` [slots, n - 1, W],
    ``gate_w`` [blocks, 2 part, part] stored as ``proj`` is (rows of r, then of i),
    ``gate_bias`` [blocks * 2 part] float32, ``softplus_lam`` [W], ``state`` [slots, W].
    Returns [T, W] as ``proj`` is stored."""
    _gpu("proj", proj, (F32, BF16), contiguous=False)
    _gpu("taps", taps, F32)
    _gpu("conv_bias", conv_bias, F32)
    _gpu("conv_state", conv_state, F32)
    _gpu("gate_w", gate_w, proj.dtype)
    _gpu("gate_bias", gate_bias, F32)
    _gpu("softplus_lam", softplus_lam, F32)
    _gpu("state", state, F32)
    _gpu("seg_pos0", seg_pos0, I32)
    _gpu("seg_slot", seg_slot, I32)
    T = proj.shape[0]
    W, n = taps.shape
    _need(gate_w.dim() == 3 and gate_w.shape[1] == 2 * gate_w.shape[2]
          and gate_w.shape[0] * gate_w.shape[2] == W,
          lambda: f"gated_unit_step: gate matrices {tuple(gate_w.shape)} for {W} channels")
    blocks, part = gate_w.shape[0], gate_w.shape[2]
    _need(proj.dim() == 2 and proj.shape[1] >= 2 * W and proj.stride(1) == 1
          and 1 <= n <= CONV_SILU_MAX_TAPS and part <= GATED_UNIT_STEP_MAX_PART
          and conv_bias.shape == (W,) and tuple(conv_state.shape[1:]) == (n - 1, W)
          and gate_bias.shape == (2 * W,) and softplus_lam.shape == (W,)
          and state.dim() == 2 and state.shape[1] == W
          and seg_pos0.shape[0] == T and seg_slot.shape[0] == T,
          lambda: f"gated_unit_step: proj {tuple(proj.shape)}, taps {tuple(taps.shape)}, "
                  f"conv_state {tuple(conv_state.shape)}, state {tuple(state.shape)}, "
                  f"{seg_slot.shape[0]} segments")
    out = torch.empty((T, W), dtype=proj.dtype, device=proj.device)
    check(library("mingru").kappai_gated_unit_step(
        _ptr(proj), _c_int(proj.stride(0)), _ptr(taps), _c_int(n), _ptr(conv_bias),
        _ptr(conv_state), _ptr(gate_w), _ptr(gate_bias), _ptr(softplus_lam), _c_float(rate),
        _ptr(state), _ptr(seg_pos0), _ptr(seg_slot), _c_int(T), _c_int(W), _c_int(blocks),
        _c_int(_is_bf16(proj.dtype)), _ptr(out), _stream()), "gated_unit_step")
    return out


# ---------------------------------------------------------------------------------------
# differential attention: the two maps of a head as heads of the paged attention kernels
# ---------------------------------------------------------------------------------------
def diff_store(proj: torch.Tensor, n_heads: int, n_kv_heads: int, dim: int, vdim: int,
               head_size: int, k_pool: torch.Tensor, v_pool: torch.Tensor, row_pos: torch.Tensor,
               row_seg: torch.Tensor, block_tables: torch.Tensor, page_size: int,
               store_kv: bool = True) -> torch.Tensor:
    """From ``proj`` [T, H 2 dim + G 2 dim + G vdim] (a head's two maps side by side): queries
    [T, 2H head_size] with map (h, m) of head h = g R + i as head (2 g + m) R + i, widened with
    zeros; keys of map m of kv head g stored as kv head 2 g + m of pools made for 2G kv heads of
    ``head_size``, the kv head's values under both."""
    H, G, d, dv, D = n_heads, n_kv_heads, dim, vdim, head_size
    _gpu("proj", proj, (F32, BF16), contiguous=False)
    T = proj.shape[0]
    need = (H * 2 * d + G * 2 * d + G * dv) if store_kv else H * 2 * d
    _need(proj.dim() == 2 and proj.shape[1] >= need and proj.stride(1) == 1,
          lambda: f"diff_store: proj {tuple(proj.shape)} holds fewer than {need} columns")
    _need(H % G == 0 and d <= D and dv <= D, lambda: f"diff_store: {H} heads over {G}, sizes "
          f"{d} and {dv} in heads of {D}")
    _gpu("row_pos", row_pos, I32)
    _gpu("row_seg", row_seg, I32)
    max_blocks = 0
    if store_kv:
        _gpu("k_pool", k_pool, proj.dtype)
        _gpu("v_pool", v_pool, proj.dtype)
        _gpu("block_tables", block_tables, I32)
        _check_pools(k_pool, v_pool, 2 * G, page_size, D)
        _need(block_tables.dim() == 2, "block_tables must be [segments, max_blocks]")
        max_blocks = block_tables.shape[1]
    q = torch.empty((T, 2 * H * D), dtype=proj.dtype, device=proj.device)
    check(library("diffattn").kappai_diff_store(
        _ptr(proj), _c_int(proj.stride(0)), _ptr(q), _ptr(k_pool), _ptr(v_pool), _ptr(row_pos),
        _ptr(row_seg), _ptr(block_tables if store_kv else None), _c_int(max_blocks), _c_int(T),
        _c_int(H), _c_int(G), _c_int(d), _c_int(dv), _c_int(D), _c_int(page_size),
        _c_int(1 if store_kv else 0), _c_int(_is_bf16(proj.dtype)), _stream()), "diff_store")
    return q


def diff_combine(ctx: torch.Tensor, n_heads: int, n_kv_heads: int, vdim: int, head_size: int,
                 lam: float, eps: float, gain: float) -> torch.Tensor:
    """``o = a1 - lam * a2`` per head from the two maps' outputs ``ctx`` [T, 2H head_size] (in
    ``diff_store``'s order), ``o / sqrt(mean(o^2) + eps) * gain`` over the head's ``vdim`` values.
    Returns [T, H vdim]."""
    H, G, dv, D = n_heads, n_kv_heads, vdim, head_size
    _gpu("ctx", ctx, (F32, BF16))
    T = ctx.shape[0]
    _need(tuple(ctx.shape) == (T, 2 * H * D), lambda: f"diff_combine: ctx {tuple(ctx.shape)}")
    out = torch.empty((T, H * dv), dtype=ctx.dtype, device=ctx.device)
    check(library("diffattn").kappai_diff_combine(
        _ptr(ctx), _ptr(out), _c_int(T), _c_int(H), _c_int(G), _c_int(dv), _c_int(D),
        _c_float(lam), _c_float(eps), _c_float(gain), _c_int(_is_bf16(ctx.dtype)), _stream()),
        "diff_combine")
    return out


# ---------------------------------------------------------------------------------------
# mixture of experts
# ---------------------------------------------------------------------------------------
MOE_MAX_TOP = 16


def moe_route(x: torch.Tensor, router: torch.Tensor, top: int,
              bias: Optional[torch.Tensor] = None):
    """Router logits ``x router^T (+ bias)`` in float32, the ``top`` largest of a row chosen (the
    lowest index wins a tie), weights = softmax over the chosen logits.  Returns (experts [T, top]
    int32, weights [T, top] float32), the largest first."""
    _gpu("x", x, (F32, BF16), contiguous=False)
    _gpu("router", router, F32)
    if bias is not None:
        _gpu("bias", bias, F32)
        _need(bias.shape == (router.shape[0],), lambda: f"moe_route: bias {tuple(bias.shape)}")
    T, D = x.shape
    E = router.shape[0]
    _need(router.shape == (E, D) and x.stride(1) == 1 and 1 <= top <= min(E, MOE_MAX_TOP),
          lambda: f"moe_route: x {tuple(x.shape)}, router {tuple(router.shape)}, top {top}")
    idx = torch.empty((T, top), dtype=I32, device=x.device)
    wts = torch.empty((T, top), dtype=F32, device=x.device)
    check(library("moe").kappai_moe_route(
        _ptr(x), _c_int(x.stride(0)), _c_int(_is_bf16(x.dtype)), _ptr(router), _ptr(bias),
        _c_int(T), _c_int(D), _c_int(E), _c_int(top), _ptr(idx), _ptr(wts), _stream()),
        "moe_route")
    return idx, wts


@dataclass
class MoePlan:
    """The step's (row, choice) pairs in expert order: ``slot_of_pair`` [T top], ``pair_of_slot``
    [tiles * tile_rows] (-1: empty), ``tile_expert`` [tiles] (-1: unused)."""
    slot_of_pair: torch.Tensor
    pair_of_slot: torch.Tensor
    tile_expert: torch.Tensor
    n_tiles: int
    tile_rows: int
    top: int


def moe_plan(experts: torch.Tensor, n_experts: int) -> MoePlan:
    _gpu("experts", experts, I32)
    T, top = experts.shape
    P = T * top
    tile = int(library("moe").kappai_moe_tile_rows())
    n_tiles = P // tile + min(n_experts, P)
    dev = experts.device
    plan = MoePlan(torch.empty((P,), dtype=I32, device=dev),
                   torch.empty((n_tiles * tile,), dtype=I32, device=dev),
                   torch.empty((n_tiles,), dtype=I32, device=dev), n_tiles, tile, top)
    check(library("moe").kappai_moe_plan(
        _ptr(experts), _c_int(P), _c_int(n_experts), _c_int(n_tiles), _ptr(plan.slot_of_pair),
        _ptr(plan.pair_of_slot), _ptr(plan.tile_expert), _stream()), "moe_plan")
    return plan


MOE_MFMA = True       # bfloat16 expert products on the matrix cores (False: the plain kernel)


MOE_FEW_PAIRS = 256   # up to this many (row, choice) pairs the expert kernels stream the matrices


class ExpertFragments:
    """The matrices of a mixture's experts [E, N, K] in the order the matrix-core kernel loads
    them: every 16 rows x 32 columns as one piece of 1 KB, lane after lane (lane = row + 16 *
    (column // 8)), the pieces of a row tile one after the other.  N a multiple of 16, K of 32."""

    def __init__(self, data: torch.Tensor, shape):
        self.data, self.shape = data, tuple(shape)
        self.dtype, self.device = data.dtype, data.device

    @staticmethod
    def fits(weight: torch.Tensor) -> bool:
        return (weight.dtype == BF16 and weight.dim() == 3 and weight.shape[1] % 16 == 0
                and weight.shape[2] % 32 == 0)

    @classmethod
    def of(cls, weight: torch.Tensor) -> "ExpertFragments":
        E, N, K = weight.shape
        w = weight.reshape(E, N // 16, 16, K // 32, 4, 8).permute(0, 1, 3, 4, 2, 5)
        return cls(w.contiguous(), (E, N, K))

    def data_ptr(self) -> int:
        return self.data.data_ptr()

    def element_size(self) -> int:
        return self.data.element_size()


def _moe_matrix(w):
    """(tensor for the checks, 1 if it lies in fragment order)"""
    return (w.data, 1) if isinstance(w, ExpertFragments) else (w, 0)


def _moe_few(plan) -> int:
    return 1 if plan.slot_of_pair.shape[0] <= MOE_FEW_PAIRS else 0


def _moe_on_matrix_cores(a: torch.Tensor, lda: int, K: int, *matrices) -> bool:
    return (MOE_MFMA and a.dtype == BF16 and K % 8 == 0 and lda % 8 == 0
            and a.data_ptr() % 16 == 0 and all(m.data_ptr() % 16 == 0 for m in matrices))


def moe_experts_gated(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor,
                      plan: MoePlan) -> torch.Tensor:
    """``silu(x Wg[e]^T) * (x Wu[e]^T)`` for every slot of the plan ([slots, F], the dtype of
    ``x``; empty slots are left unwritten).  ``w_gate``, ``w_up``: [E, F, D]."""
    _gpu("x", x, (F32, BF16), contiguous=False)
    E, F, D = w_gate.shape
    (w_gate, frag), (w_up, frag_up) = _moe_matrix(w_gate), _moe_matrix(w_up)
    _gpu("w_gate", w_gate, x.dtype)
    _gpu("w_up", w_up, x.dtype)
    _need(w_up.shape == w_gate.shape and frag == frag_up and x.shape[1] == D
          and x.stride(1) == 1,
          lambda: f"moe_experts_gated: x {tuple(x.shape)}, matrices {(E, F, D)}")
    out = torch.empty((plan.n_tiles * plan.tile_rows, F), dtype=x.dtype, device=x.device)
    mfma = _moe_on_matrix_cores(x, x.stride(0), D, w_gate, w_up)
    _need(mfma or not frag, "moe_experts_gated: matrices in fragment order need bfloat16 rows "
          "with 16-byte aligned starts")
    if mfma:
        check(library("moe").kappai_moe_gemm_mfma(
            _ptr(x), _c_int(x.stride(0)), _ptr(w_gate), _ptr(w_up), _c_int(F), _c_int(D),
            _ptr(plan.tile_expert), _ptr(plan.pair_of_slot), _c_int(plan.top),
            _c_int(plan.n_tiles), _ptr(out), _c_int(1), _c_int(_moe_few(plan)), _c_int(frag),
            _stream()), "moe_gemm_mfma (gate, up)")
        return out
    check(library("moe").kappai_moe_gemm(
        _ptr(x), _c_int(x.stride(0)), _ptr(w_gate), _ptr(w_up), _c_int(F), _c_int(D),
        _ptr(plan.tile_expert), _ptr(plan.pair_of_slot), _c_int(plan.top), _c_int(plan.n_tiles),
        _ptr(out), _c_int(1), _c_int(_is_bf16(x.dtype)), _stream()), "moe_gemm (gate, up)")
    return out


def moe_experts_activated(x: torch.Tensor, w_up: torch.Tensor, plan: MoePlan) -> torch.Tensor:
    """``relu(x Wu[e]^T)^2`` for every slot of the plan ([slots, F], the dtype of ``x``; empty
    slots are left unwritten): experts of one matrix in, no gate.  ``w_up``: [E, F, D]."""
    _gpu("x", x, (F32, BF16), contiguous=False)
    E, F, D = w_up.shape
    w_up, frag = _moe_matrix(w_up)
    _gpu("w_up", w_up, x.dtype)
    _need(x.shape[1] == D and x.stride(1) == 1,
          lambda: f"moe_experts_activated: x {tuple(x.shape)}, matrices {(E, F, D)}")
    out = torch.empty((plan.n_tiles * plan.tile_rows, F), dtype=x.dtype, device=x.device)
    mfma = _moe_on_matrix_cores(x, x.stride(0), D, w_up)
    _need(mfma or not frag, "moe_experts_activated: matrices in fragment order need bfloat16 "
          "rows with 16-byte aligned starts")
    if mfma:
        check(library("moe").kappai_moe_gemm_mfma(
            _ptr(x), _c_int(x.stride(0)), _ptr(w_up), _vp(0), _c_int(F), _c_int(D),
            _ptr(plan.tile_expert), _ptr(plan.pair_of_slot), _c_int(plan.top),
            _c_int(plan.n_tiles), _ptr(out), _c_int(2), _c_int(_moe_few(plan)), _c_int(frag),
            _stream()), "moe_gemm_mfma (up, squared relu)")
        return out
    check(library("moe").kappai_moe_gemm(
        _ptr(x), _c_int(x.stride(0)), _ptr(w_up), _vp(0), _c_int(F), _c_int(D),
        _ptr(plan.tile_expert), _ptr(plan.pair_of_slot), _c_int(plan.top), _c_int(plan.n_tiles),
        _ptr(out), _c_int(2), _c_int(_is_bf16(x.dtype)), _stream()),
        "moe_gemm (up, squared relu)")
    return out


def moe_experts_down(act: torch.Tensor, w_down: torch.Tensor, plan: MoePlan) -> torch.Tensor:
    """``act W_down[e]^T`` for every slot of the plan: float32 [slots, D]."""
    _gpu("act", act, (F32, BF16))
    E, D, F = w_down.shape
    w_down, frag = _moe_matrix(w_down)
    _gpu("w_down", w_down, act.dtype)
    _need(tuple(act.shape) == (plan.n_tiles * plan.tile_rows, F),
          lambda: f"moe_experts_down: act {tuple(act.shape)}, matrices {(E, D, F)}")
    out = torch.empty((act.shape[0], D), dtype=F32, device=act.device)
    mfma = _moe_on_matrix_cores(act, F, F, w_down)
    _need(mfma or not frag, "moe_experts_down: matrices in fragment order need bfloat16 rows")
    if mfma:
        check(library("moe").kappai_moe_gemm_mfma(
            _ptr(act), _c_int(F), _ptr(w_down), _vp(0), _c_int(D), _c_int(F),
            _ptr(plan.tile_expert), _ptr(plan.pair_of_slot), _c_int(plan.top),
            _c_int(plan.n_tiles), _ptr(out), _c_int(0), _c_int(_moe_few(plan)), _c_int(frag),
            _stream()), "moe_gemm_mfma (down)")
        return out
    check(library("moe").kappai_moe_gemm(
        _ptr(act), _c_int(F), _ptr(w_down), _vp(0), _c_int(D), _c_int(F),
        _ptr(plan.tile_expert), _ptr(plan.pair_of_slot), _c_int(plan.top), _c_int(plan.n_tiles),
        _ptr(out), _c_int(0), _c_int(_is_bf16(act.dtype)), _stream()), "moe_gemm (down)")
    return out


def moe_combine(y: torch.Tensor, weights: torch.Tensor, plan: MoePlan,
                also: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out[t] = (also[t] +) sum_k weights[t, k] * y[slot of (t, k)]`` in the order of k: float32
    [T, D].  ``also``: what every row gets beside its experts, [T, D] in float32 or bfloat16, or
    float32 partial sums [S, T, D] (added in order)."""
    _gpu("y", y, F32)
    _gpu("weights", weights, F32)
    T, top = weights.shape
    D = y.shape[1]
    _need(top == plan.top and plan.slot_of_pair.shape[0] == T * top, "moe_combine: another plan")
    parts = 1
    if also is not None:
        _gpu("also", also, (F32, BF16))
        if also.dim() == 3:
            _need(also.dtype == F32, "moe_combine: partial sums are float32")
            parts = also.shape[0]
        _need(tuple(also.shape[-2:]) == (T, D), lambda: f"moe_combine: also {tuple(also.shape)}")
    out = torch.empty((T, D), dtype=F32, device=y.device)
    check(library("moe").kappai_moe_combine(
        _ptr(y), _ptr(plan.slot_of_pair), _ptr(weights), _c_int(T), _c_int(top), _c_int(D),
        _ptr(also), _c_int(_is_bf16(also.dtype) if also is not None else 0), _c_int(parts),
        _ptr(out), _stream()), "moe_combine")
    return out


# ---------------------------------------------------------------------------------------
# a norm on a sublayer's output, added into the residual stream
# ---------------------------------------------------------------------------------------
def output_norm_add(resid: torch.Tensor, a: torch.Tensor, weight: torch.Tensor, eps: float,
                    rows_dtype=None, scale_a: float = 1.0, b: Optional[torch.Tensor] = None,
                    scale_b: float = 1.0, add: bool = True) -> Optional[torch.Tensor]:
    """``y = scale_a a (+ scale_b b)``; ``resid (+)= y / sqrt(mean(y^2) + eps) * weight`` in
    float32, in place (``add`` False: the residual becomes the normalised rows).  ``a``: [T, D]
    in float32 or bfloat16, or float32 partial sums [S, T, D], added in order first; ``b`` like
    ``a`` but always [T, D].  With ``rows_dtype`` the new residual is also returned rounded to that
    dtype, for the next sublayer to read."""
    _gpu("resid", resid, F32)
    _gpu("a", a, (F32, BF16))
    _gpu("weight", weight, F32)
    T, D = resid.shape
    parts = 1
    if a.dim() == 3:
        _need(a.dtype == F32, "output_norm_add: partial sums are float32")
        parts = a.shape[0]
    _need(tuple(a.shape[-2:]) == (T, D) and weight.shape == (D,),
          lambda: f"output_norm_add: {tuple(a.shape)} into {tuple(resid.shape)}")
    if b is not None:
        _gpu("b", b, a.dtype)
        _need(tuple(b.shape) == (T, D), lambda: f"output_norm_add: b {tuple(b.shape)}")
    rows = None
    if rows_dtype is not None:
        rows = torch.empty((T, D), dtype=rows_dtype, device=resid.device)
    check(library("elementwise").kappai_output_norm_add(
        _ptr(a), _c_int(_is_bf16(a.dtype)), _c_int(parts), _c_float(scale_a), _ptr(b),
        _c_float(scale_b), _ptr(weight), _c_float(eps), _ptr(resid), _c_int(1 if add else 0),
        _ptr(rows), _c_int(_is_bf16(rows_dtype) if rows is not None else 0), _c_int(T), _c_int(D),
        _stream()), "output_norm_add")
    return rows


def pair_norm_sum(a: torch.Tensor, b: torch.Tensor, scale_a: float = 1.0, scale_b: float = 1.0,
                  weight_a: Optional[torch.Tensor] = None,
                  weight_b: Optional[torch.Tensor] = None, eps: float = 0.0) -> torch.Tensor:
    """``scale_a * n_a(a) + scale_b * n_b(b)`` in float32, ``n(y) = y / sqrt(mean(y^2) + eps) * w``
    where a weight [D] is given and ``y`` itself where not.  ``a``, ``b`` [T, D] in one dtype
    (float32 or bfloat16).  Returns float32 [T, D]."""
    _gpu("a", a, (F32, BF16))
    _gpu("b", b, a.dtype)
    _need(a.dim() == 2 and a.shape == b.shape, lambda: f"pair_norm_sum: {tuple(a.shape)} and "
                                                       f"{tuple(b.shape)}")
    T, D = a.shape
    for name, w in (("weight_a", weight_a), ("weight_b", weight_b)):
        if w is not None:
            _gpu(name, w, F32)
            _need(w.shape == (D,), lambda: f"pair_norm_sum: {name} {tuple(w.shape)}")
    out = torch.empty((T, D), dtype=F32, device=a.device)
    check(library("elementwise").kappai_pair_norm_sum(
        _ptr(a), _c_float(scale_a), _ptr(weight_a), _ptr(b), _c_float(scale_b), _ptr(weight_b),
        _c_float(eps), _c_int(T), _c_int(D), _ptr(out), _c_int(_is_bf16(a.dtype)), _stream()),
        "pair_norm_sum")
    return out


def stream_enter(resid: torch.Tensor, delta: Optional[torch.Tensor],
                 again: Optional[torch.Tensor], row: Optional[torch.Tensor]) -> None:
    """``resid += delta`` (a pending update [T, D], float32 or bfloat16, or None), ``+= again``
    (float32 [T, D] or None), ``+= row`` (float32 [D] or None), in this order, in place."""
    _gpu("resid", resid, F32)
    T, D = resid.shape
    if delta is not None:
        _gpu("delta", delta, (F32, BF16))
        _need(tuple(delta.shape) == (T, D), lambda: f"stream_enter: delta {tuple(delta.shape)}")
    if again is not None:
        _gpu("again", again, F32)
        _need(tuple(again.shape) == (T, D), lambda: f"stream_enter: again {tuple(again.shape)}")
    if row is not None:
        _gpu("row", row, F32)
        _need(tuple(row.shape) == (D,), lambda: f"stream_enter: row {tuple(row.shape)}")
    check(library("elementwise").kappai_stream_enter(
        _ptr(resid), _ptr(delta), _c_int(_is_bf16(delta.dtype) if delta is not None else 0),
        _ptr(again), _ptr(row), _c_int(T), _c_int(D), _stream()), "stream_enter")


# ---------------------------------------------------------------------------------------
# attention layers whose queries, keys and values are not the plain grouped-query form
# ---------------------------------------------------------------------------------------
def projection_norm_store(proj: torch.Tensor, n_heads: int, n_kv_heads: int, dim: int, vdim: int,
                          head_size: int, q_norm_w: Optional[torch.Tensor],
                          k_norm_w: Optional[torch.Tensor], eps: float, temp_coef: float,
                          temp_every: int, k_pool: torch.Tensor, v_pool: torch.Tensor,
                          row_pos: torch.Tensor, row_seg: torch.Tensor,
                          block_tables: torch.Tensor, page_size: int,
                          store_kv: bool = True) -> torch.Tensor:
    """From ``proj`` [T, H dim + G dim + G vdim]: q and k each divided by the root mean square of
    their WHOLE projection (all heads together) and multiplied by weights [H dim] / [G dim]
    (None: no norm); q also by ``1 + temp_coef * ln(floor((position + 1) / temp_every) + 1)``.
    Returns queries [T, H head_size] (zeros behind ``dim``); keys and values go to pools made for
    G kv heads of ``head_size`` (``PagedKV``)."""
    H, G, d, dv, D = n_heads, n_kv_heads, dim, vdim, head_size
    _gpu("proj", proj, (F32, BF16), contiguous=False)
    T = proj.shape[0]
    need = H * d + G * d + G * dv
    _need(proj.dim() == 2 and proj.shape[1] >= need and proj.stride(1) == 1,
          lambda: f"projection_norm_store: proj {tuple(proj.shape)} holds fewer than {need} columns")
    _need(H % G == 0 and d <= D and dv <= D and temp_every >= 1,
          lambda: f"projection_norm_store: {H} heads over {G}, sizes {d} and {dv} in heads of {D}")
    for name, w, n in (("q_norm_w", q_norm_w, H * d), ("k_norm_w", k_norm_w, G * d)):
        if w is not None:
            _gpu(name, w, F32)
            _need(w.shape == (n,), lambda: f"{name}: {tuple(w.shape)}, expected ({n},)")
    _gpu("row_pos", row_pos, I32)
    _gpu("row_seg", row_seg, I32)
    max_blocks = 0
    if store_kv:
        _gpu("k_pool", k_pool, proj.dtype)
        _gpu("v_pool", v_pool, proj.dtype)
        _gpu("block_tables", block_tables, I32)
        _check_pools(k_pool, v_pool, G, page_size, D)
        max_blocks = block_tables.shape[1]
    q = torch.empty((T, H * D), dtype=proj.dtype, device=proj.device)
    check(library("attn_prep").kappai_projection_norm_store(
        _ptr(proj), _c_int(proj.stride(0)), _ptr(q_norm_w), _ptr(k_norm_w), _c_float(eps),
        _c_float(temp_coef), _c_int(temp_every), _ptr(k_pool if store_kv else None),
        _ptr(v_pool if store_kv else None), _ptr(row_pos), _ptr(row_seg),
        _ptr(block_tables if store_kv else None), _c_int(max_blocks), _c_int(T), _c_int(H),
        _c_int(G), _c_int(d), _c_int(dv), _c_int(D), _c_int(page_size), _ptr(q),
        _c_int(_is_bf16(proj.dtype)), _stream()), "projection_norm_store")
    return q


def rotate_widen_store(proj: torch.Tensor, n_heads: int, n_kv_heads: int, dim: int, vdim: int,
                       head_size: int, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
                       rot_dims: int, rot_mode: int, values_are_keys: bool,
                       k_pool: torch.Tensor, v_pool: torch.Tensor, row_pos: torch.Tensor,
                       row_seg: torch.Tensor, block_tables: torch.Tensor,
                       page_size: int) -> torch.Tensor:
    """From ``proj`` [T, H dim + G dim (+ G vdim)]: the first ``rot_dims`` places of every q and
    k head turn by the row's position (``cos`` / ``sin`` [positions, rot_dims / 2] float32, with
    whatever factor the encoding puts on them; ``rot_mode`` as ``qk_norm_rope_store``).  Returns
    queries [T, H head_size] (zeros behind ``dim``); keys and values go to pools made for G kv
    heads of ``head_size``.  ``values_are_keys``: there are no value columns; a kv head's value
    is its key as projected, before the rotation."""
    H, G, d, dv, D = n_heads, n_kv_heads, dim, vdim, head_size
    _gpu("proj", proj, (F32, BF16), contiguous=False)
    T = proj.shape[0]
    need = H * d + G * d + (0 if values_are_keys else G * dv)
    _need(proj.dim() == 2 and proj.shape[1] >= need and proj.stride(1) == 1,
          lambda: f"rotate_widen_store: proj {tuple(proj.shape)} holds fewer than {need} columns")
    _need(H % G == 0 and d <= D and dv <= D and (not values_are_keys or dv == d),
          lambda: f"rotate_widen_store: {H} heads over {G}, sizes {d} and {dv} in heads of {D}")
    if rot_mode != ROT_NONE and rot_dims:
        _gpu("cos", cos, F32)
        _gpu("sin", sin, F32)
        _need(rot_dims % 2 == 0 and rot_dims <= d and cos.shape == sin.shape and cos.dim() == 2
              and cos.shape[1] == rot_dims // 2,
              lambda: f"rotate_widen_store: tables {tuple(cos.shape)} for {rot_dims} places of {d}")
    else:
        rot_dims, rot_mode, cos, sin = 0, ROT_NONE, None, None
    _gpu("k_pool", k_pool, proj.dtype)
    _gpu("v_pool", v_pool, proj.dtype)
    _check_pools(k_pool, v_pool, G, page_size, D)
    for name, t in (("row_pos", row_pos), ("row_seg", row_seg), ("block_tables", block_tables)):
        _gpu(name, t, I32)
    _need(row_pos.shape[0] == T and row_seg.shape[0] == T and block_tables.dim() == 2,
          "rotate_widen_store: row tables do not fit the batch")
    q = torch.empty((T, H * D), dtype=proj.dtype, device=proj.device)
    check(library("attn_prep").kappai_rotate_widen_store(
        _ptr(proj), _c_int(proj.stride(0)), _ptr(cos), _ptr(sin), _c_int(rot_dims),
        _c_int(rot_mode), _c_int(1 if values_are_keys else 0), _ptr(k_pool), _ptr(v_pool),
        _ptr(row_pos), _ptr(row_seg), _ptr(block_tables), _c_int(block_tables.shape[1]),
        _c_int(T), _c_int(H), _c_int(G), _c_int(d), _c_int(dv), _c_int(D), _c_int(page_size),
        _ptr(q), _c_int(_is_bf16(proj.dtype)), _stream()), "rotate_widen_store")
    return q


def head_norm_rotate_store(proj: torch.Tensor, n_heads: int, n_kv_heads: int, dim: int,
                           vdim: int, head_size: int, q_norm_w: Optional[torch.Tensor],
                           k_norm_w: Optional[torch.Tensor], eps: float,
                           cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
                           rot_dims: int, rot_mode: int, k_pool: torch.Tensor,
                           v_pool: torch.Tensor, row_pos: torch.Tensor, row_seg: torch.Tensor,
                           block_tables: torch.Tensor, page_size: int) -> torch.Tensor:
    """From ``proj`` [T, H dim + G dim + G vdim (+ more)]: every q and k head divided by the root
    mean square of its own ``dim`` places and multiplied by a weight [dim] that the heads share
    (None: no norm), then the first ``rot_dims`` places turned by the row's position (tables and
    ``rot_mode`` as ``rotate_widen_store``).  Returns queries [T, H head_size] (zeros behind
    ``dim``); keys and values go to pools made for G kv heads of ``head_size``."""
    H, G, d, dv, D = n_heads, n_kv_heads, dim, vdim, head_size
    _gpu("proj", proj, (F32, BF16), contiguous=False)
    T = proj.shape[0]
    need = H * d + G * d + G * dv
    _need(proj.dim() == 2 and proj.shape[1] >= need and proj.stride(1) == 1,
          lambda: f"head_norm_rotate_store: proj {tuple(proj.shape)} holds fewer than {need} "
                  "columns")
    _need(H % G == 0 and d <= D and dv <= D,
          lambda: f"head_norm_rotate_store: {H} heads over {G}, sizes {d} and {dv} in heads of {D}")
    for name, w in (("q_norm_w", q_norm_w), ("k_norm_w", k_norm_w)):
        if w is not None:
            _gpu(name, w, F32)
            _need(w.shape == (d,), lambda: f"{name}: {tuple(w.shape)}, expected ({d},)")
    if rot_mode != ROT_NONE and rot_dims:
        _gpu("cos", cos, F32)
        _gpu("sin", sin, F32)
        _need(rot_dims % 2 == 0 and rot_dims <= d and cos.shape == sin.shape and cos.dim() == 2
              and cos.shape[1] == rot_dims // 2,
              lambda: f"head_norm_rotate_store: tables {tuple(cos.shape)} for {rot_dims} places "
                      f"of {d}")
    else:
        rot_dims, rot_mode, cos, sin = 0, ROT_NONE, None, None
    _gpu("k_pool", k_pool, proj.dtype)
    _gpu("v_pool", v_pool, proj.dtype)
    _check_pools(k_pool, v_pool, G, page_size, D)
    for name, t in (("row_pos", row_pos), ("row_seg", row_seg), ("block_tables", block_tables)):
        _gpu(name, t, I32)
    _need(row_pos.shape[0] == T and row_seg.shape[0] == T and block_tables.dim() == 2,
          "head_norm_rotate_store: row tables do not fit the batch")
    q = torch.empty((T, H * D), dtype=proj.dtype, device=proj.device)
    check(library("attn_prep").kappai_head_norm_rotate_store(
        _ptr(proj), _c_int(proj.stride(0)), _ptr(q_norm_w), _ptr(k_norm_w), _c_float(eps),
        _ptr(cos), _ptr(sin), _c_int(rot_dims), _c_int(rot_mode), _ptr(k_pool), _ptr(v_pool),
        _ptr(row_pos), _ptr(row_seg), _ptr(block_tables), _c_int(block_tables.shape[1]),
        _c_int(T), _c_int(H), _c_int(G), _c_int(d), _c_int(dv), _c_int(D), _c_int(page_size),
        _ptr(q), _c_int(_is_bf16(proj.dtype)), _stream()), "head_norm_rotate_store")
    return q


def latent_store(q: torch.Tensor, kv: torch.Tensor, n_heads: int, dim: int, rot_dim: int,
                 rank: int, head_size: int, c_norm_w: torch.Tensor, eps: float,
                 cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], rot_dims: int,
                 rot_mode: int, k_pool: torch.Tensor, v_pool: torch.Tensor,
                 row_pos: torch.Tensor, row_seg: torch.Tensor, block_tables: torch.Tensor,
                 page_size: int) -> torch.Tensor:
    """``kv`` [T, rank + rot_dim]: the first ``rank`` entries, RMS-normed with ``c_norm_w``, are
    the token's latent; the rest is a key part that is rotated by the position.  They are stored
    as the one kv head's key ``[latent | rotated | 0]`` of ``head_size``, the latent again as its
    value.  ``q`` [T, H (dim + rot_dim)], head by head ``[dim | rot_dim]``: returns
    [T, H head_size] whose places ``rank .. rank + rot_dim`` of every head hold the rotated part
    (zeros behind); the first ``rank`` places are left for ``headwise_linear``."""
    H, d, rot, r, D = n_heads, dim, rot_dim, rank, head_size
    _gpu("q", q, (F32, BF16), contiguous=False)
    _gpu("kv", kv, q.dtype, contiguous=False)
    T = q.shape[0]
    _need(q.dim() == 2 and q.shape[1] >= H * (d + rot) and q.stride(1) == 1 and kv.dim() == 2
          and kv.shape[0] == T and kv.shape[1] >= r + rot and kv.stride(1) == 1,
          lambda: f"latent_store: q {tuple(q.shape)}, kv {tuple(kv.shape)}")
    _need(D >= r + rot and rot_dims <= rot and rot_dims % 2 == 0,
          lambda: f"latent_store: a latent of {r} and {rot} rotated places in heads of {D}")
    _gpu("c_norm_w", c_norm_w, F32)
    _need(c_norm_w.shape == (r,), "latent_store: one norm weight for each entry of the latent")
    if rot_mode != ROT_NONE and rot_dims:
        _gpu("cos", cos, F32)
        _gpu("sin", sin, F32)
        _need(cos.shape == sin.shape and cos.dim() == 2 and cos.shape[1] == rot_dims // 2,
              lambda: f"latent_store: rotation tables {tuple(cos.shape)} for {rot_dims} places")
    _gpu("k_pool", k_pool, q.dtype)
    _gpu("v_pool", v_pool, q.dtype)
    _check_pools(k_pool, v_pool, 1, page_size, D)
    for name, t in (("row_pos", row_pos), ("row_seg", row_seg), ("block_tables", block_tables)):
        _gpu(name, t, I32)
    out = torch.empty((T, H * D), dtype=q.dtype, device=q.device)
    check(library("attn_prep").kappai_latent_store(
        _ptr(q), _c_int(q.stride(0)), _ptr(kv), _c_int(kv.stride(0)), _ptr(c_norm_w),
        _c_float(eps), _ptr(cos), _ptr(sin), _c_int(rot_dims), _c_int(rot_mode), _ptr(k_pool),
        _ptr(v_pool), _ptr(row_pos), _ptr(row_seg), _ptr(block_tables),
        _c_int(block_tables.shape[1]), _c_int(T), _c_int(H), _c_int(d), _c_int(rot), _c_int(r),
        _c_int(D), _c_int(page_size), _ptr(out), _c_int(_is_bf16(q.dtype)), _stream()),
        "latent_store")
    return out


def headwise_linear(x: torch.Tensor, x_head_stride: int, weight: torch.Tensor,
                    out: Optional[torch.Tensor] = None, out_head_stride: Optional[int] = None,
                    out_dtype=None, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``y[t, h, :] = weight[h] @ x[t, h, :]`` with ``weight`` [H, n_out, n_in] in the dtype of
    ``x``.  ``out_dtype`` float32 keeps the sums as they are (else they are stored as ``x`` is).  Head h of row t starts at ``x[t, h * x_head_stride]`` and is written at
    ``out[t, h * out_head_stride]`` (``out`` None: a new [T, H n_out]).  ``gate`` [T, H n_out] in
    the dtype of ``x`` (rows may be strided): every result is multiplied by the sigmoid of its
    gate before it is stored."""
    _gpu("x", x, (F32, BF16), contiguous=False)
    _gpu("weight", weight, x.dtype)
    _need(weight.dim() == 3, "headwise_linear: weight must be [heads, out, in]")
    H, n_out, n_in = weight.shape
    T = x.shape[0]
    _need(x.dim() == 2 and x.stride(1) == 1 and (H - 1) * x_head_stride + n_in <= x.shape[1],
          lambda: f"headwise_linear: x {tuple(x.shape)} for {H} heads of {n_in} every "
                  f"{x_head_stride}")
    out_dtype = x.dtype if out_dtype is None else out_dtype
    _need(out_dtype in (x.dtype, F32), "headwise_linear: results as x is stored, or float32")
    if out is None:
        out = torch.empty((T, H * n_out), dtype=out_dtype, device=x.device)
        out_head_stride = n_out
    _gpu("out", out, out_dtype, contiguous=False)
    _need(out.dim() == 2 and out.shape[0] == T and out.stride(1) == 1
          and (H - 1) * out_head_stride + n_out <= out.shape[1],
          lambda: f"headwise_linear: out {tuple(out.shape)}")
    if gate is not None:
        _gpu("gate", gate, x.dtype, contiguous=False)
        _need(gate.dim() == 2 and gate.shape[0] == T and gate.shape[1] >= H * n_out
              and gate.stride(1) == 1, lambda: f"headwise_linear: gate {tuple(gate.shape)}")
    check(library("attn_prep").kappai_headwise_linear(
        _ptr(x), _c_int(x.stride(0)), _c_int(x_head_stride), _ptr(weight), _c_int(H),
        _c_int(n_out), _c_int(n_in), _ptr(out), _c_int(out.stride(0)), _c_int(out_head_stride),
        _c_int(T), _c_int(_is_bf16(x.dtype)), _c_int(1 if out_dtype == F32 else 0), _ptr(gate),
        _c_int(gate.stride(0) if gate is not None else 0), _stream()), "headwise_linear")
    return out


# ---------------------------------------------------------------------------------------
# recurrences with a matrix of state per head
# ---------------------------------------------------------------------------------------
CONV_SILU_MAX_TAPS = 17


def conv_silu(x: torch.Tensor, taps: torch.Tensor, state: torch.Tensor, row_pos: torch.Tensor,
              row_seg: torch.Tensor, seg_start: torch.Tensor, seg_pos0: torch.Tensor,
              seg_slot: torch.Tensor, bias: Optional[torch.Tensor] = None,
              activation: bool = True) -> torch.Tensor:
    """``silu(conv(x) + bias)`` per channel (``activation`` False: no SiLU; ``bias`` [C] float32
    or None): ``conv(x)[t] = sum_j taps[:, j] x[t - n + 1 + j]``, zeros
    before position 0.  ``x`` [T, >= C] (a view with a row stride), ``taps`` [C, n] float32,
    ``state`` [slots, n - 1, C] float32: the request's last inputs, read for rows before the
    step's portion and brought up to date.  Returns [T, C] in the dtype of ``x``."""
    _gpu("x", x, (F32, BF16), contiguous=False)
    _gpu("taps", taps, F32)
    _gpu("state", state, F32)
    C, n = taps.shape
    T = x.shape[0]
    _need(x.dim() == 2 and x.shape[1] >= C and x.stride(1) == 1,
          lambda: f"conv_silu: x {tuple(x.shape)} for {C} channels")
    _need(1 <= n <= CONV_SILU_MAX_TAPS and tuple(state.shape[1:]) == (n - 1, C),
          lambda: f"conv_silu: {n} taps, state {tuple(state.shape)}")
    for name, t in (("row_pos", row_pos), ("row_seg", row_seg), ("seg_start", seg_start),
                    ("seg_pos0", seg_pos0), ("seg_slot", seg_slot)):
        _gpu(name, t, I32)
    S = seg_slot.shape[0]
    if bias is not None:
        _gpu("bias", bias, F32)
        _need(bias.shape == (C,), lambda: f"conv_silu: bias {tuple(bias.shape)} for {C} channels")
    out = torch.empty((T, C), dtype=x.dtype, device=x.device)
    check(library("linear_attention").kappai_conv_silu(
        _ptr(x), _c_int(x.stride(0)), _ptr(taps), _c_int(n), _ptr(state), _ptr(row_pos),
        _ptr(row_seg), _ptr(seg_start), _ptr(seg_pos0), _ptr(seg_slot), _c_int(T), _c_int(S),
        _c_int(C), _ptr(bias), _c_int(1 if activation else 0), _ptr(out),
        _c_int(_is_bf16(x.dtype)), _stream()), "conv_silu")
    return out


def token_shift_mix(h: torch.Tensor, mu: torch.Tensor, state: torch.Tensor,
                    row_pos: torch.Tensor, row_seg: torch.Tensor, seg_start: torch.Tensor,
                    seg_slot: torch.Tensor) -> torch.Tensor:
    """``out[m] = h + (h' - h) * mu[m]`` with ``h'`` the row of the token before (zeros at position
    0): ``h`` [T, W], ``mu`` [n, W] float32, ``state`` [slots, W] float32 (the request's last row,
    read for a segment's first row and brought up to date).  Returns [n, T, W] as ``h`` is stored."""
    _gpu("h", h, (F32, BF16), contiguous=False)
    _gpu("mu", mu, F32)
    _gpu("state", state, F32)
    T, W = h.shape
    _need(h.stride(1) == 1 and mu.dim() == 2 and mu.shape[1] == W
          and tuple(state.shape[1:]) == (W,),
          lambda: f"token_shift_mix: h {tuple(h.shape)}, mu {tuple(mu.shape)}, state "
                  f"{tuple(state.shape)}")
    for name, t in (("row_pos", row_pos), ("row_seg", row_seg), ("seg_start", seg_start),
                    ("seg_slot", seg_slot)):
        _gpu(name, t, I32)
    S = seg_slot.shape[0]
    out = torch.empty((mu.shape[0], T, W), dtype=h.dtype, device=h.device)
    check(library("linear_attention").kappai_token_shift_mix(
        _ptr(h), _c_int(h.stride(0)), _ptr(mu), _c_int(mu.shape[0]), _ptr(state), _ptr(row_pos),
        _ptr(row_seg), _ptr(seg_start), _ptr(seg_slot), _c_int(T), _c_int(S), _c_int(W),
        _ptr(out), _c_int(_is_bf16(h.dtype)), _stream()), "token_shift_mix")
    return out


SCAN_FORMS = {"auto": 0, "wave": 1, "block": 2}


DECAY_KINDS = {"softplus": 0, "double_exp": 1, "fixed": 2}
FIXED_DECAY_CHUNK_ROWS = 32     # the most rows of a chunk the chunked form of a fixed decay takes


def matrix_state_recurrence(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                            z: Optional[torch.Tensor],
                            n_heads: int, n_qk_heads: int, dim: int, vdim: int,
                            rate: Optional[torch.Tensor], z_bias: Optional[torch.Tensor],
                            z_sign: float,
                            q_scale: float, state: torch.Tensor, seg_start: torch.Tensor,
                            seg_pos0: torch.Tensor, seg_slot: torch.Tensor,
                            beta: Optional[torch.Tensor] = None, unit_qk: bool = False,
                            unit_eps: float = 1e-6, form: str = "auto",
                            decay: str = "softplus", bonus: Optional[torch.Tensor] = None,
                            silu_inputs: bool = False, chunks: Optional[torch.Tensor] = None,
                            seg_chunk0: Optional[torch.Tensor] = None,
                            chunk_rows: int = 0) -> torch.Tensor:
    """A state ``S`` [dim, vdim] per head, float32, kept column by column in ``state``
    [slots, H, vdim, dim] (a segment that starts at position 0 starts from zero).  Per token, with the decay per key channel
    ``a = exp(-rate[h] * softplus(z_sign * (z + z_bias)))``:
    without ``beta``   ``S <- diag(a) S + k v^T``, ``o = S^T q``;
    with ``beta``      ``S <- diag(a) S``, ``u = sigmoid(beta) (v - S^T k)``, ``S <- S + k u^T``,
                       ``o = S^T q`` (the delta rule; the read-out sees the token's own write);
    with ``bonus``     ``o = (S + diag(bonus[h]) k v^T)^T q``, then ``S <- diag(a) S + k v^T`` (the
                       read-out sees the state before the token, and the token itself weighed by
                       ``bonus`` [H, dim] float32).
    ``decay`` = "double_exp": ``a = exp(-exp(z + z_bias))``; "fixed": ``a = rate[h]`` for every
    token and channel (``z`` None).  ``silu_inputs``: q, k and v pass SiLU first (rounded as they
    are stored).
    ``q``, ``k`` [T, Hk dim] (head h reads q/k head ``h // (H / Hk)``; ``unit_qk``: each head's
    vector divided by ``sqrt(sum x^2 + unit_eps)`` first), q times ``q_scale``; ``v`` [T, H vdim];
    ``z`` [T, H dim]; ``beta`` [T, H]; all views with a row stride.  Everything between the
    projections and the result is float32.  Returns ``o`` [T, H vdim] float32.

    ``form`` = "wave" | "block" forces one of the two kernels (for tests): a wave that reads each
    token from global memory, or a block of waves that takes the tokens in chunks through LDS.

    ``chunks`` [n, 3] = (segment, first row, rows <= ``chunk_rows`` <= 32) with ``seg_chunk0``
    [S + 1], as for ``mingru_scan``: a fixed decay (no ``beta``, no ``bonus``, H == Hk) and the
    form with a ``bonus`` are then worked chunk by chunk in three passes, with no chain along the
    tokens of a chunk (every factor is a product of decays, none is divided by one)."""
    H, Hk, d, dv = n_heads, n_qk_heads, dim, vdim
    _need(form in SCAN_FORMS, lambda: f"matrix_state_recurrence: form {form!r}")
    _need(decay in DECAY_KINDS and (z is None) == (decay == "fixed")
          and (rate is not None or decay == "double_exp"),
          lambda: f"matrix_state_recurrence: decay {decay!r} with z {'given' if z is not None else 'missing'}")
    _need(beta is None or bonus is None, "matrix_state_recurrence: the delta rule or a bonus")
    _need(not (silu_inputs and unit_qk), "matrix_state_recurrence: SiLU or unit vectors")
    T = q.shape[0]
    for name, t, cols in (("q", q, Hk * d), ("k", k, Hk * d), ("v", v, H * dv), ("z", z, H * d)):
        if t is None:
            continue
        _gpu(name, t, q.dtype, contiguous=False)
        _need(t.dim() == 2 and t.shape[0] == T and t.shape[1] >= cols and t.stride(1) == 1,
              lambda: f"matrix_state_recurrence: {name} {tuple(t.shape)}, expected [T, {cols}]")
    _need(q.dtype in (F32, BF16) and H % Hk == 0, "matrix_state_recurrence: dtypes / heads")
    if beta is not None:
        _gpu("beta", beta, q.dtype, contiguous=False)
        _need(beta.dim() == 2 and beta.shape[0] == T and beta.shape[1] >= H
              and (beta.stride(1) == 1 or H == 1), "matrix_state_recurrence: beta must be [T, H]")
    if rate is not None:
        _gpu("rate", rate, F32)
        _need(rate.shape == (H,), "matrix_state_recurrence: one rate a head")
    if bonus is not None:
        _gpu("bonus", bonus, F32)
        _need(tuple(bonus.shape) == (H, d) and H == Hk,
              lambda: f"matrix_state_recurrence: bonus {tuple(bonus.shape)} for {H} heads of {d}")
    if z_bias is not None:
        _gpu("z_bias", z_bias, F32)
        _need(z_bias.shape == (H * d,), "matrix_state_recurrence: z_bias must be [H dim]")
    _gpu("state", state, F32)
    _need(tuple(state.shape[1:]) == (H, dv, d),
          lambda: f"matrix_state_recurrence: state {tuple(state.shape)} for {H} x {dv} x {d}")
    for name, t in (("seg_start", seg_start), ("seg_pos0", seg_pos0), ("seg_slot", seg_slot)):
        _gpu(name, t, I32)
    S = seg_slot.shape[0]
    dev = q.device
    qf = torch.empty((T, Hk * d), dtype=F32, device=dev)
    kf = torch.empty((T, Hk * d), dtype=F32, device=dev)
    af = torch.empty((T, H * d), dtype=F32, device=dev)
    bf = torch.empty((T, H), dtype=F32, device=dev) if beta is not None else None
    vf = torch.empty((T, H * dv), dtype=F32, device=dev) if silu_inputs else None
    lib = library("linear_attention")
    check(lib.kappai_recurrence_prep(
        _ptr(q), _c_int(q.stride(0)), _ptr(k), _c_int(k.stride(0)), _ptr(z),
        _c_int(z.stride(0) if z is not None else 0),
        _ptr(z_bias), _ptr(rate), _c_float(z_sign), _ptr(beta),
        _c_int(beta.stride(0) if beta is not None else 0), _c_int(T), _c_int(H), _c_int(Hk),
        _c_int(d), _c_int(1 if unit_qk else 0), _c_float(unit_eps), _c_float(q_scale),
        _c_int(1 if silu_inputs else 0), _c_int(DECAY_KINDS[decay]),
        _ptr(v if silu_inputs else None), _c_int(v.stride(0)), _c_int(dv), _ptr(qf),
        _ptr(kf), _ptr(af), _ptr(bf), _ptr(vf), _c_int(_is_bf16(q.dtype)), _stream()),
        "recurrence_prep")
    out = torch.empty((T, H * dv), dtype=F32, device=dev)
    values = vf if silu_inputs else v
    mode = 1 if beta is not None else 2 if bonus is not None else 0
    if chunks is not None and H == Hk and ((decay == "fixed" and mode == 0) or mode == 2):
        _gpu("chunks", chunks, I32)
        _gpu("seg_chunk0", seg_chunk0, I32)
        _need(chunks.dim() == 2 and chunks.shape[1] == 3 and seg_chunk0.shape[0] == S + 1
              and 1 <= chunk_rows <= FIXED_DECAY_CHUNK_ROWS,
              lambda: f"matrix_state_recurrence: chunk tables {tuple(chunks.shape)} of "
                      f"{chunk_rows} rows do not fit")
        n_chunks = chunks.shape[0]
        carry = torch.empty((n_chunks, H, dv, d), dtype=F32, device=dev)
        if mode == 2:
            total = torch.empty((n_chunks, H, d), dtype=F32, device=dev)
            check(lib.kappai_channel_decay_chunks(
                _ptr(qf), _ptr(kf), _ptr(af), _ptr(values), _c_int(values.stride(0)),
                _c_int(_is_bf16(values.dtype)), _ptr(bonus), _ptr(state), _ptr(seg_pos0),
                _ptr(seg_slot), _ptr(chunks), _ptr(seg_chunk0), _c_int(n_chunks),
                _c_int(chunk_rows), _c_int(T), _c_int(S), _c_int(H), _c_int(d), _c_int(dv),
                _ptr(carry), _ptr(total), _ptr(out), _stream()), "channel_decay_chunks")
            return out
        check(lib.kappai_fixed_decay_chunks(
            _ptr(qf), _ptr(kf), _ptr(values), _c_int(values.stride(0)),
            _c_int(_is_bf16(values.dtype)), _ptr(rate), _ptr(state), _ptr(seg_pos0),
            _ptr(seg_slot), _ptr(chunks), _ptr(seg_chunk0), _c_int(n_chunks), _c_int(chunk_rows),
            _c_int(T), _c_int(S), _c_int(H), _c_int(d), _c_int(dv), _ptr(carry), _ptr(out),
            _stream()), "fixed_decay_chunks")
        return out
    check(lib.kappai_matrix_state_scan(
        _ptr(qf), _ptr(kf), _ptr(af), _ptr(bonus if bonus is not None else bf), _ptr(values),
        _c_int(values.stride(0)),
        _c_int(_is_bf16(values.dtype)), _ptr(state), _ptr(seg_start), _ptr(seg_pos0),
        _ptr(seg_slot),
        _c_int(T), _c_int(S), _c_int(H), _c_int(Hk), _c_int(d), _c_int(dv),
        _c_int(mode), _c_int(SCAN_FORMS[form]), _ptr(out), _stream()),
        "matrix_state_scan")
    return out


GATE_SILU, GATE_SIGMOID = 0, 1


def head_norm_gate(o: torch.Tensor, weight: torch.Tensor, eps: float, gate: torch.Tensor,
                   gate_kind: int, n_heads: int, vdim: int, out_dtype) -> torch.Tensor:
    """Per head ``o / sqrt(mean(o^2) + eps) * weight`` (``weight`` [vdim], shared by the heads, or
    [H, vdim], one a head) times ``silu(gate)`` or ``sigmoid(gate)``: ``o`` [T, H vdim] float32, ``gate`` [T, >= H vdim]
    in ``out_dtype`` (a view with a row stride).  Returns [T, H vdim] in ``out_dtype``."""
    H, dv = n_heads, vdim
    _gpu("o", o, F32)
    _gpu("weight", weight, F32)
    _gpu("gate", gate, out_dtype, contiguous=False)
    T = o.shape[0]
    _need(tuple(o.shape) == (T, H * dv) and tuple(weight.shape) in ((dv,), (H, dv))
          and gate.dim() == 2
          and gate.shape[0] == T and gate.shape[1] >= H * dv and gate.stride(1) == 1,
          lambda: f"head_norm_gate: o {tuple(o.shape)}, gate {tuple(gate.shape)}")
    out = torch.empty((T, H * dv), dtype=out_dtype, device=o.device)
    check(library("linear_attention").kappai_head_norm_gate(
        _ptr(o), _ptr(weight), _c_float(eps), _ptr(gate), _c_int(gate.stride(0)),
        _c_int(gate_kind), _c_int(T), _c_int(H), _c_int(dv),
        _c_int(dv if weight.dim() == 2 else 0), _ptr(out),
        _c_int(_is_bf16(out_dtype)), _stream()), "head_norm_gate")
    return out


# ---------------------------------------------------------------------------------------
# a residual stream kept in several copies, its layer norm, gates and caps
# ---------------------------------------------------------------------------------------
HYPER_MAX_STREAMS = 8


def hyper_step(streams: Optional[torch.Tensor], n_streams: int, width: int, source=None, y=None,
               mix=None, out_w=None, in_w=None, norm_w=None, eps: float = 0.0, rows=None,
               rows_dtype=None, store: bool = True) -> Optional[torch.Tensor]:
    """One pass over the copies of the stream, ``streams`` [T, S, W] float32, in place.

    Write half (``y``, ``mix`` [S, S] indexed [from, to], ``out_w`` [S]): every copy becomes
    ``x_t <- sum_s mix[s, t] x_s + out_w[t] * y``, all from the old copies; ``y`` is [T, W] in
    float32 or bfloat16, or float32 partial sums [P, T, W] added in order.  Read half (``in_w``
    [S], ``norm_w`` [W], ``rows_dtype``): ``u = sum_s in_w[s] x_s`` of the new copies passes a
    layer norm without bias, ``(u - mean) / sqrt(var + eps) * norm_w``, and is returned as
    [T, W] in ``rows_dtype``.  ``source`` [T, W]: the copies do not exist yet and are all this
    row (they are then written to ``streams`` when ``store``).  ``rows`` (int32): the read half
    runs for these rows only, and the new copies are not stored."""
    S, W = n_streams, width
    _need(1 <= S <= HYPER_MAX_STREAMS, lambda: f"hyper_step: {S} copies of the stream; the kernel "
                                               f"takes 1 to {HYPER_MAX_STREAMS}")
    if streams is not None:
        _gpu("streams", streams, F32)
        _need(streams.dim() == 3 and tuple(streams.shape[1:]) == (S, W),
              lambda: f"hyper_step: streams {tuple(streams.shape)} for {S} copies of {W}")
    if source is not None:
        _gpu("source", source, F32)
        _need(source.dim() == 2 and source.shape[1] == W,
              lambda: f"hyper_step: source {tuple(source.shape)}")
    _need(streams is not None or source is not None, "hyper_step: nothing to read")
    T = streams.shape[0] if streams is not None else source.shape[0]
    _need(source is None or streams is None or source.shape[0] == T, "hyper_step: source rows")
    parts = 1
    if y is not None:
        _gpu("y", y, (F32, BF16))
        if y.dim() == 3:
            _need(y.dtype == F32, "hyper_step: partial sums are float32")
            parts = y.shape[0]
        _need(tuple(y.shape[-2:]) == (T, W), lambda: f"hyper_step: y {tuple(y.shape)}")
        _gpu("mix", mix, F32)
        _gpu("out_w", out_w, F32)
        _need(tuple(mix.shape) == (S, S) and tuple(out_w.shape) == (S,),
              lambda: f"hyper_step: mix {tuple(mix.shape)}, out {tuple(out_w.shape)}")
    normed = None
    n_rows = T
    if rows is not None:
        _gpu("rows", rows, I32)
        n_rows = rows.shape[0]
        store = False
    if rows_dtype is not None:
        _gpu("in_w", in_w, F32)
        _gpu("norm_w", norm_w, F32)
        _need(tuple(in_w.shape) == (S,) and tuple(norm_w.shape) == (W,),
              lambda: f"hyper_step: in {tuple(in_w.shape)}, norm weight {tuple(norm_w.shape)}")
        normed = torch.empty((n_rows, W), dtype=rows_dtype, device=(
            streams if streams is not None else source).device)
    store = bool(store and streams is not None and (y is not None or source is not None))
    check(library("streams").kappai_hyper_step(
        _ptr(streams), _ptr(source), _ptr(y), _c_int(_is_bf16(y.dtype) if y is not None else 0),
        _c_int(parts), _ptr(mix if y is not None else None),
        _ptr(out_w if y is not None else None), _ptr(in_w if normed is not None else None),
        _ptr(norm_w if normed is not None else None), _c_float(eps), _ptr(rows), _c_int(n_rows),
        _c_int(1 if store else 0), _ptr(normed),
        _c_int(_is_bf16(rows_dtype) if normed is not None else 0), _c_int(T), _c_int(S),
        _c_int(W), _stream()), "hyper_step")
    return normed


def rows_rmsnorm(x: torch.Tensor, n: int, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """The first ``n`` columns of every row of ``x`` (rows may be strided) divided by their root
    mean square (eps inside the root) and multiplied by ``weight`` [n]: a new [T, n] as ``x`` is
    stored; sums in float32."""
    _gpu("x", x, (F32, BF16), contiguous=False)
    _gpu("weight", weight, F32)
    _need(x.dim() == 2 and x.stride(1) == 1 and 1 <= n <= x.shape[1] and weight.shape == (n,),
          lambda: f"rows_rmsnorm: x {tuple(x.shape)}, {n} columns, weight {tuple(weight.shape)}")
    out = torch.empty((x.shape[0], n), dtype=x.dtype, device=x.device)
    check(library("streams").kappai_rows_rmsnorm(
        _ptr(x), _c_int(x.stride(0)), _ptr(weight), _c_float(eps), _c_int(x.shape[0]), _c_int(n),
        _ptr(out), _c_int(_is_bf16(x.dtype)), _stream()), "rows_rmsnorm")
    return out


def sigmoid_gate(x: torch.Tensor, gate: torch.Tensor, group: int) -> torch.Tensor:
    """``x[t, i] *= sigmoid(gate[t, i // group])`` in place; ``x`` [T, n] contiguous, ``gate``
    [T, n / group] in the same dtype (rows may be strided).  ``group`` 1: a gate a channel; the
    head size: a gate a head."""
    _gpu("x", x, (F32, BF16))
    _gpu("gate", gate, x.dtype, contiguous=False)
    T, n = x.shape
    _need(group >= 1 and n % group == 0 and gate.dim() == 2 and gate.shape[0] == T
          and gate.shape[1] >= n // group and gate.stride(1) == 1,
          lambda: f"sigmoid_gate: x {tuple(x.shape)}, gate {tuple(gate.shape)}, groups of {group}")
    check(library("streams").kappai_sigmoid_gate(
        _ptr(x), _ptr(gate), _c_int(gate.stride(0)), _c_int(T), _c_int(n), _c_int(group),
        _c_int(_is_bf16(x.dtype)), _stream()), "sigmoid_gate")
    return x


def softcap_rows(x: torch.Tensor, cap: float) -> torch.Tensor:
    """``x <- cap * tanh(x / cap)`` in place; float32."""
    _gpu("x", x, F32)
    _need(cap > 0.0, lambda: f"softcap_rows: a cap of {cap}")
    check(library("streams").kappai_softcap_rows(_ptr(x), _c_long(x.numel()), _c_float(cap),
                                                 _stream()), "softcap_rows")
    return x


ACT_RELU_SQUARED = 0


def activate(x: torch.Tensor, kind: int = ACT_RELU_SQUARED) -> torch.Tensor:
    """An activation without a gate on every element, stored as ``x`` is: ``ACT_RELU_SQUARED``,
    ``relu(x)^2``."""
    _gpu("x", x, (F32, BF16))
    _need(kind == ACT_RELU_SQUARED, lambda: f"activate: unknown activation {kind}")
    out = torch.empty_like(x)
    check(library("streams").kappai_activate(
        _ptr(x), _ptr(out), _c_long(x.numel()), _c_int(kind), _c_int(_is_bf16(x.dtype)),
        _stream()), "activate")
    return out
