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
                  weight_frag: Optional[torch.Tensor] = None, out_fragment: bool = False):
    """``silu(x Wg^T) * (x Wu^T)`` in one kernel: ``weight`` [2F, K] holds the gate and up
    matrices interleaved by ``interleave_gate_up``; bfloat16 only.  Returns [M, F].  ``x`` may
    be ``ScaledRows`` or ``FragmentRows``.  ``out_fragment``: with 8 to 16 rows the result may
    come back as ``FragmentRows`` for the product that follows."""
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
    check(library("gemm").kappai_gemm_bf16_swiglu(
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


def decode_form(n_heads: int, n_kv_heads: int, head_dim: int, max_position: int,
                window: int = 0) -> str:
    """Which of the two decode kernels a step takes: with few keys ("decode-block") a block per
    (row, kv head) splits them over its waves and merges in LDS; else ("decode-split") the keys
    are split over blocks, whose partial results a second kernel merges."""
    n_keys = min(max_position + 1, window) + 32 if window else max_position + 1
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
                    max_lone_position: int = -1) -> torch.Tensor:
    """Causal attention of every row over the keys of its request that are in the cache
    (its own included; the last ``window`` of them when a window is set).  ``q`` is
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
    through the decode kernel that splits keys over blocks."""
    H, G, d = n_heads, n_kv_heads, head_dim
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
        check(library("attention").kappai_paged_attention_rows(
            _ptr(q), _c_int(q.stride(0)), _ptr(k_pool), _ptr(v_pool), _ptr(out), _c_int(H * d),
            _ptr(row_pos), _ptr(row_seg), _ptr(block_tables), _c_int(block_tables.shape[1]),
            _c_int(T), _c_int(H), _c_int(G), _c_int(d), _c_int(page_size), _c_int(window or 0),
            _c_float(scale), _c_int(_is_bf16(q.dtype)), _stream()), "paged_attention_rows")
        return out
    _need(mfma_ok, "the matrix-core attention kernels need bfloat16, a page size and a head size "
          f"that are multiples of 16 (head size at most 256) and 16-byte aligned rows; got "
          f"{q.dtype}, page {page_size}, head {d}")
    lib = library("attention_mfma", HEAD_DIM=d)
    if kernel == "prefill":
        _gpu("q_tiles", q_tiles, I32)
        _need(q_tiles.dim() == 2 and q_tiles.shape[1] == 4, "q_tiles must be [tiles, 4]")
        check(lib.kappai_attn_prefill(
            _ptr(q), _c_int(q.stride(0)), _ptr(k_pool), _ptr(v_pool), _ptr(out), _c_int(H * d),
            _ptr(q_tiles), _c_int(q_tiles.shape[0]), _ptr(row_pos), _ptr(block_tables),
            _c_int(block_tables.shape[1]), _c_int(H), _c_int(G), _c_int(page_size),
            _c_int(window or 0), _c_float(scale), _c_int(prefill_variant), _stream()),
            "attn_prefill")
        if lone_rows is not None:
            _gpu("lone_rows", lone_rows, I32)
            _need(H // G <= 16 and lone_rows.dim() == 1 and max_lone_position >= 0,
                  "paged_attention: rows left out of the tiles need the decode kernel (at most 16 "
                  "query heads a kv head) and their largest position")
            _decode_split(lib, q, H, G, d, k_pool, v_pool, row_pos, row_seg, block_tables,
                          page_size, scale, window, max_lone_position, out, lone_rows)
        return out
    _need(kernel in ("decode", "decode-block", "decode-split"),
          lambda: f"unknown attention kernel {kernel!r}")
    _need(H // G <= 16, "the decode kernel takes at most 16 query heads per kv head")
    _need(max_position is not None, "the decode kernel needs the batch's largest position")
    qk_args = ()
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
    n_keys = min(max_position + 1, window) + 32 if window else max_position + 1
    block_waves = lib.kappai_attn_decode_block_waves(H // G)
    if kernel == "decode":
        kernel = "decode-split" if qk is not None else decode_form(H, G, d, max_position, window)
    if kernel == "decode-block":
        _need(block_waves > 0, "too many query heads a kv head for the block form")
        _need(qk is None, "the decode kernel that keeps a row's keys in one block takes q ready "
                          "made and the keys stored")
        check(lib.kappai_attn_decode_block(
            _ptr(q), _c_int(q.stride(0)), _ptr(k_pool), _ptr(v_pool), _ptr(out), _c_int(H * d),
            _ptr(row_pos), _ptr(row_seg), _ptr(block_tables), _c_int(block_tables.shape[1]),
            _c_int(T), _c_int(H), _c_int(G), _c_int(page_size), _c_int(window or 0),
            _c_float(scale), _c_int(block_waves), _stream()), "attn_decode_block")
        return out
    _decode_split(lib, q, H, G, d, k_pool, v_pool, row_pos, row_seg, block_tables, page_size, scale,
                  window, max_position, out, None, qk_args)
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
                  window, max_position, out, row_ids, qk_args=()):
    """The decode kernel that splits a row's keys over blocks, and its merge, for all rows or
    (``row_ids``) some of them."""
    T = q.shape[0] if row_ids is None else row_ids.shape[0]
    n_keys = min(max_position + 1, window) + 32 if window else max_position + 1
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
    if row_ids is not None:
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
