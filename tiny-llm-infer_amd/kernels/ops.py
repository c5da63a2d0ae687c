"""The kernel library as the parts see it: hand-written HIP kernels for gfx950,
called through a C ABI on torch tensors.  There is no CPU path and no
fallback: without the library, or without a GPU, construction fails.

Every wrapper checks on the host that shapes, dtypes and devices are what the
kernel and its grid assume before anything is launched.
"""
from __future__ import annotations

import contextlib
import ctypes
from ctypes import c_float, c_int, c_void_p
from typing import Optional, Tuple

import torch

from . import build

F32, BF16 = 0, 1


class KernelError(RuntimeError):
    pass


class PendingProduct:
    """x W^T not run yet: what ``linear(..., deferred=True)`` returns for a decode step's
    few rows.  ``add_rmsnorm(..., lazy=True)`` runs it with the residual sum and the
    norm taken into the product; anything else runs it as it is (``resolve``)."""

    def __init__(self, x: torch.Tensor, matrix):
        self.x, self.matrix = x, matrix
        self.shape = (x.shape[0], _shape_of(matrix)[0])
        self.dtype = x.dtype


class NormedRows:
    """Rows of a norm whose scalar factor is still owed: ``xw`` = bfloat16(weight * h)
    [rows, n] and ``ssq`` [parts, rows], partial sums of h^2 in float32; the normed rows
    are xw / sqrt(sum(ssq) / n + eps).  ``linear`` and ``linear_swiglu`` take it as their
    input and apply the factor to their outputs."""

    def __init__(self, xw: torch.Tensor, ssq: torch.Tensor, eps: float):
        self.xw, self.ssq, self.eps = xw, ssq, float(eps)
        self.shape = tuple(xw.shape)
        self.dtype = xw.dtype


def _dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"kernels take float32 or bfloat16 tensors, not {dtype}")


_LIB = None


def load_library():
    """Load (building it first if nothing is built) the shared library."""
    global _LIB
    if _LIB is not None:
        return _LIB
    path = build.find_library() or build.build_library()
    try:
        lib = ctypes.CDLL(path)
    except OSError as exc:
        raise KernelError(f"cannot load the kernel library {path}: {exc}") from None
    lib.tli_last_error.restype = ctypes.c_char_p
    P, I, F = c_void_p, c_int, c_float
    sigs = {
        "tli_abi_version": [],
        "tli_device_compute_units": [],
        "tli_embed": [P, P, P, I, I, I, I, P],
        "tli_feed_tokens": [P, P, P, I, I, P],
        "tli_add_rmsnorm": [P, P, P, P, P, I, I, I, F, I, I, P],
        "tli_swiglu": [P, P, I, I, I, P],
        "tli_qkv_to_cache": [P, P, P, P, P, P, P, I, I, I, I, I, I, I, P, F, P, F, P, P, I, I, I, I, I, P],
        "tli_values_to_cache": [P, P, P, P, I, I, P, I, I, I, I, I, I, P],
        "tli_keys_values_to_cache": [P, P, P, P, P, I, I, P, I, I, I, I, I, I, P, F, P, P, I, P],
        "tli_attention_plain": [P, P, P, P, P, P, P, I, I, I, I, I, I, I, F, I, I, P],
        "tli_gemm_plain": [P, P, P, I, I, I, I, I, I, P],
        "tli_gemm_skinny_bf16": [P, P, P, I, I, I, I, I, I, P],
        "tli_gemm_skinny_fused_bf16": [P, P, P, I, I, I, I, P, I, F, P, P, P, P, I, P],
        "tli_gemm_mid_bf16": [P, P, P, P, I, I, I, I, I, I, I, P],
        "tli_gemm_mid_splits": [I, I, I],
        "tli_gemm_mid_splits_rows": [I, I, I, I],
        "tli_gemm_mid_reduce": [P, P, I, I, I, I, P],
        "tli_gemm_rows_bf16": [P, P, P, P, I, I, I, I, I, I, P],
        "tli_gemm_rows_splits": [I, I, I],
        "tli_attention_decode_bf16": [P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, F, I, I, I, P],
        "tli_qkv_attention_decode_bf16": [P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, P, F, P, F, P, P, I,
                                          F, I, I, I, P, I, P],
        "tli_attention_prefill_bf16": [P, P, P, P, P, P, I, I, P, I, I, I, I, I, I, F, I, I, P],
        "tli_qkv_attention_prefill_bf16": [P, P, P, P, P, P, I, I, P, I, I, I, I, I, I, P, F, P, P, F, I, I, P],
        "tli_sample": [P, I, I, P, P, P, P, P, P],
        "tli_sample_scratch_bytes": [I],
        "tli_random_normal": [P, ctypes.c_longlong, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, P, F, F, I, P],
    }
    for name, args in sigs.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = c_int
    lib.tli_sample_uniform.argtypes = [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32]
    lib.tli_sample_uniform.restype = c_float
    _LIB = lib
    return lib


def _shape_of(w) -> Tuple[int, int]:
    """(out, in) of a [out, in] tensor or of a matrix as the parts hold it, without asking for its
    row-major form (which such a matrix may have to put together first)."""
    shape = getattr(w, "shape", None)
    return tuple(shape) if shape is not None else tuple(w.w.shape)


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


class DeferredSum:
    """A matrix product whose k range was split, left as float32 partial sums
    [splits, rows, cols].  ``HipOps.linear(..., deferred=True)`` may return one
    instead of a tensor; ``add_rmsnorm`` takes it as the delta and adds the parts
    itself (rounding the sum to ``dtype`` as the product's own reduction would),
    anything else calls ``HipOps.resolve`` first."""

    def __init__(self, parts: torch.Tensor, dtype: torch.dtype):
        self.parts = parts
        self.dtype = dtype
        self.shape = tuple(parts.shape[1:])


class HipOps:
    name = "hip-gfx950"
    MAX_HEAD_DIM = 512
    SKINNY_ROWS = 64
    MID_ROWS_FROM = 17           # from this many rows the x-sharing kernel multiplies,
    MID_ROWS_TO = 128            # up to this many
    MID_ROWS_TO_PLAIN = 256      # a product without a gate: up to this many (two blocks of 128 rows side by side)
    DECODE_WORKGROUPS = 256      # the device's compute units (set to what the device reports when the library is loaded):
                                 # the decode attention splits a row's keys to come near one workgroup for each
    DECODE_SPLIT_KEYS = 1024     # a split walks at least this many keys
    # A step of prompt portions whose first sequences decode: the prefill kernel takes a row that decodes
    # as a sequence of one row, beside its other workgroups; the decode kernel is a second launch (8 to 10
    # us) that runs before it, but splits a long row's keys and puts four waves on a row.  Those rows go
    # to the decode kernel when they are few and much longer than the portions (up to 8 rows of 3,000
    # keys and more, twice the longest portion's sequence: 4 rows of 4,000 keys beside 256 / 1,024 /
    # 2,000 new tokens 62 / 110 / 126 us in the prefill kernel, 47 / 69 / 98 us with the decode kernel),
    # or many beside short portions (64 rows and more beside at most 512 new tokens: 64 rows of 200 keys
    # beside 256 tokens 50 against 42 us, 128 rows 75 against 53).  Measured at 4 to 128 rows of 200 to
    # 4,000 keys beside 256 to 2,000 new tokens behind up to 3,584 keys; elsewhere the prefill kernel
    # alone is as fast or up to a fifth faster.
    DECODE_BESIDE_FEW = (8, 3000, 2.0)       # at most so many rows, of at least so many keys and so many times the portions' longest
    DECODE_BESIDE_MANY = (64, 512)           # at least so many rows, beside at most so many new tokens

    def __init__(self, device):
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise KernelError(f"the kernels run on an AMD GPU ('cuda:N' in torch), not on '{device}'")
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible to torch; this engine has no CPU path")
        self.lib = load_library()
        with torch.cuda.device(self.device):
            self.DECODE_WORKGROUPS = int(self.lib.tli_device_compute_units())
        self._held_stream = None
        self.force_plain = False     # tests: run the plain attention kernel for bfloat16 too
        self.plain_products = False  # every matrix product through the plain kernel
        self.separate_norms = False  # tests: decode steps run their norms as kernels of their own
        self.unfused_decode = False  # tests: decode steps through qkv_to_cache and paged_attention too
        self.separate_cache_writes = False   # tests: the keys and the values of prompt portions by a kernel each
        self.decode_solo = "auto"    # the decode attention that gives a row's kv head a wave to itself: "auto" (where
                                     # the rows fill the chip), "always" (wherever its limits allow), "never"
        self.prefill_direct = 0      # tests: 1 = the prefill attention kernel without LDS staging; 2, 3 = with, 1 or 2 tiles a wave; 4..8 = a forced order of row blocks; 10, 11 = heads of 64 and 128 with two sets of waves a workgroup, with one; 13 = as 0 for rows with many keys before them
        self.mid_cfg = 0             # measurements: launch shape and k ranges of the 17..128-row kernel
        self.mid_splits = 0
        self.skinny_cfg = 0          # measurements: force a launch shape of the weight-streaming kernel
        # Products of more than 128 rows: "own" = gemm_rows; "library" = the BLAS library; "measure" = the
        # faster of the two for the shape, timed once when the shape first comes up.  The latter two
        # multiply with the row-major form of a matrix, which is then held beside its decode layout
        # (see keep_row_major): set this before the weights are loaded.
        self.many_rows = "own"
        self.measured = {}           # (rows rounded up to 128, N, K, gated) -> True where gemm_rows won
        self._cold = None            # what is written between two timed runs
        self.rows_cfg = 0            # measurements: force a launch shape and the k ranges of gemm_rows
        self.rows_splits = 0

    @property
    def keep_row_major(self) -> bool:
        """Whether a bfloat16 matrix is to keep its row-major form beside its decode layout."""
        return self.many_rows != "own"

    def use_plain_kernels(self) -> None:
        """Every product, attention and norm through the plain kernels, bfloat16 too
        (what the float32 path runs): to tell a fault of a tuned kernel from one elsewhere."""
        self.force_plain = self.plain_products = self.separate_norms = self.unfused_decode = True

    # ---- helpers ----------------------------------------------------------
    def _stream(self):
        if self._held_stream is not None:
            return self._held_stream
        return torch.cuda.current_stream(self.device).cuda_stream

    @contextlib.contextmanager
    def hold_stream(self):
        """Inside, every kernel goes to the stream that was current on entry: one look-up for the
        hundreds of launches of a step instead of one each (a quarter of the host's time in a step
        that is not replayed from a recording)."""
        before = self._held_stream
        self._held_stream = torch.cuda.current_stream(self.device).cuda_stream
        try:
            yield
        finally:
            self._held_stream = before

    def _call(self, fn, *args):
        if fn(*args) != 0:
            raise KernelError(self.lib.tli_last_error().decode())

    def _want(self, t: torch.Tensor, what: str, dtype=None, shape=None):
        if t.device != self.device:
            raise KernelError(f"{what} is on {t.device}, expected {self.device}")
        if not t.is_contiguous():
            raise KernelError(f"{what} must be contiguous")
        if dtype is not None and t.dtype != dtype:
            raise KernelError(f"{what} has dtype {t.dtype}, expected {dtype}")
        if shape is not None and tuple(t.shape) != tuple(shape):
            raise KernelError(f"{what} has shape {tuple(t.shape)}, expected {tuple(shape)}")

    # ---- limits that parts ask about at build time --------------------------
    def check_attention_sizes(self, heads: int, kv_heads: int, head_dim: int) -> None:
        if head_dim % 16 or not 16 <= head_dim <= self.MAX_HEAD_DIM:
            raise KernelError(f"head_dim {head_dim} is not supported: the attention kernels take "
                              f"multiples of 16 from 16 to {self.MAX_HEAD_DIM}")
        if heads <= 0 or kv_heads <= 0 or heads % kv_heads:
            raise KernelError(f"{heads} heads cannot be grouped over {kv_heads} kv heads")

    def check_page_size(self, page_size: int) -> None:
        if page_size <= 0 or page_size > 256 or page_size & (page_size - 1):
            raise KernelError(f"page size {page_size} is not supported: powers of two up to 256")

    # ---- ops ------------------------------------------------------------------
    def feed_tokens(self, token_ids: torch.Tensor, token_from: torch.Tensor, src: torch.Tensor, rows: int):
        """token_ids[r] = src[token_from[r]] where token_from[r] >= 0 (all int32, on the device)."""
        for t, what in ((token_ids, "token ids"), (token_from, "token sources"), (src, "sampled tokens")):
            self._want(t, what, torch.int32)
        if token_ids.numel() < rows or token_from.numel() < rows:
            raise KernelError("fewer token ids than rows")
        self._call(self.lib.tli_feed_tokens, token_ids.data_ptr(), token_from.data_ptr(), src.data_ptr(),
                   rows, src.numel(), self._stream())

    def embed(self, table: torch.Tensor, token_ids: torch.Tensor, num_rows: int) -> torch.Tensor:
        vocab, hidden = table.shape
        self._want(table, "embedding table")
        self._want(token_ids, "token ids", torch.int32)
        if token_ids.numel() < num_rows:
            raise KernelError("fewer token ids than rows")
        out = torch.empty((num_rows, hidden), dtype=torch.float32, device=self.device)
        self._call(self.lib.tli_embed, table.data_ptr(), token_ids.data_ptr(), out.data_ptr(),
                   num_rows, hidden, vocab, _dtype_code(table.dtype), self._stream())
        return out

    def resolve(self, y):
        """The tensor of a product that ``linear(..., deferred=True)`` left unfinished."""
        if isinstance(y, PendingProduct):
            return self.linear(y.x, y.matrix)
        if isinstance(y, NormedRows):
            raise KernelError("normed rows that still owe their factor go to linear or linear_swiglu")
        if not isinstance(y, DeferredSum):
            return y
        splits, M, N = y.parts.shape
        out = torch.empty((M, N), dtype=y.dtype, device=self.device)
        self._call(self.lib.tli_gemm_mid_reduce, y.parts.data_ptr(), out.data_ptr(), M, N, splits,
                   _dtype_code(y.dtype), self._stream())
        return out

    def add_rmsnorm(self, resid, delta, weight, eps, out_dtype, rows=None, num_rows=None, lazy=False):
        """``lazy``: the caller hands the result to ``linear`` or ``linear_swiglu`` only and so
        also takes ``NormedRows``."""
        total, n = resid.shape
        self._want(resid, "residual", torch.float32)
        self._want(weight, "norm weight", torch.float32, (n,))
        if isinstance(delta, PendingProduct):
            if lazy and rows is None and not self.separate_norms:
                return self._product_into_residual(delta, resid, weight, eps)
            delta = self.resolve(delta)
        parts = 0
        if isinstance(delta, DeferredSum):
            if delta.dtype != out_dtype or out_dtype != torch.bfloat16:
                delta = self.resolve(delta)
            else:
                parts = delta.parts.shape[0]
                delta = delta.parts
                self._want(delta, "partial sums of the residual delta", torch.float32, (parts, total, n))
        if delta is not None and not parts:
            self._want(delta, "residual delta", out_dtype, (total, n))
        out_rows = total
        if rows is not None:
            self._want(rows, "row list", torch.int32)
            out_rows = rows.numel() if num_rows is None else num_rows
            if rows.numel() < out_rows:
                raise KernelError("row list is shorter than the rows asked for")
        out = torch.empty((out_rows, n), dtype=out_dtype, device=self.device)
        self._call(self.lib.tli_add_rmsnorm, resid.data_ptr(), _ptr(delta), weight.data_ptr(),
                   out.data_ptr(), _ptr(rows), out_rows, total, n, float(eps),
                   _dtype_code(out_dtype), parts, self._stream())
        return out

    def tile_matrix(self, w: torch.Tensor) -> Optional[torch.Tensor]:
        """The decode layout of a bfloat16 matrix W[N,K]: blocks of 16 rows x 128
        columns, zero-padded to whole blocks, stored [row block][column block][j][lane][8]
        with lane = 16*c + r holding W[16*row block + r][128*column block + 32*c + 8*j + e].
        A wave of the weight-streaming kernel then reads 4 KiB in a row per block, in the
        order its MFMA operands want.  None if the matrix cannot use that kernel."""
        N, K = w.shape
        if w.dtype != torch.bfloat16 or K % 8:
            return None
        n16, k128 = (N + 15) // 16 * 16, (K + 127) // 128 * 128
        if (n16, k128) != (N, K):
            padded = torch.zeros((n16, k128), dtype=w.dtype, device=w.device)
            padded[:N, :K] = w
            w = padded
        t = w.view(n16 // 16, 16, k128 // 128, 4, 4, 8)          # [nb, r, kb, c, j, e]
        return t.permute(0, 2, 4, 3, 1, 5).contiguous()           # [nb, kb, j, c, r, e]

    def untile_matrix(self, tiled: torch.Tensor, shape) -> torch.Tensor:
        """The row-major matrix [N, K] again from its decode layout (a new tensor)."""
        N, K = shape
        nb, kb = tiled.shape[0], tiled.shape[1]
        w = tiled.permute(0, 4, 1, 3, 2, 5).reshape(nb * 16, kb * 128)        # [nb, r, kb, c, j, e]
        return w[:N, :K].contiguous()

    def linear(self, x: torch.Tensor, w, out_dtype: Optional[torch.dtype] = None, deferred: bool = False,
               sums_only: bool = False):
        """y = x W^T.  ``w`` is a [N, K] tensor or a ``Matrix`` (row-major tensor plus
        its decode layout).  ``deferred``: the caller hands the result to ``add_rmsnorm``
        (or to ``resolve``) and so also takes a ``PendingProduct`` or a ``DeferredSum``;
        ``sums_only``: to ``qkv_attention`` (or to ``resolve``), which takes a ``DeferredSum``."""
        if isinstance(x, NormedRows):
            return self._linear_normed(x, w, getattr(w, "tiled", None), 0, out_dtype)
        if self.plain_products:
            return self.linear_plain(x, getattr(w, "w", w), out_dtype)
        tiled = getattr(w, "tiled", None)
        if (deferred and not sums_only and tiled is not None and x.dtype == torch.bfloat16
                and 0 < x.shape[0] <= 16 and out_dtype in (None, torch.bfloat16) and not self.separate_norms):
            return PendingProduct(x, w)
        matrix = w
        M, K = x.shape
        N, K2 = _shape_of(matrix)
        if K != K2:
            raise KernelError(f"linear: input has {K} columns, the matrix {K2}")
        self._want(x, "linear input")
        w_dtype = getattr(matrix, "dtype", None) or matrix.w.dtype
        if x.dtype != w_dtype:
            raise KernelError(f"linear: input is {x.dtype}, the matrix {w_dtype}")
        out_dtype = out_dtype or x.dtype
        y = torch.empty((M, N), dtype=out_dtype, device=self.device)
        if M == 0:
            return y
        if x.dtype == torch.bfloat16 and K % 8 == 0:
            # (beyond 128 rows only with bfloat16 results, and not where the library or a measurement was asked for)
            if tiled is not None and self.MID_ROWS_FROM <= M <= (
                    self.MID_ROWS_TO_PLAIN if out_dtype == torch.bfloat16 and self.many_rows == "own" else self.MID_ROWS_TO):
                return self._linear_mid(x, tiled, y, M, N, K, 0, deferred or sums_only)
            if tiled is not None and out_dtype == torch.float32 and M > self.MID_ROWS_TO:
                # float32 logits for many rows (a decode step of hundreds of requests, a replay that wants
                # every position): the x-sharing kernel, 256 rows (two row blocks side by side) at a time
                # (512 rows of the Qwen3-8B head: 8 x 363 us in the kernel below, 4 x 240 us in portions of
                # 128 rows).  The last rows too, however few: a row's sums are then the same bits whatever
                # the number of rows beside it in its block of 128, which a step replayed with rows that
                # only fill it up relies on.
                for m0 in range(0, M, self.MID_ROWS_TO_PLAIN):
                    m1 = min(M, m0 + self.MID_ROWS_TO_PLAIN)
                    self._linear_mid(x[m0:m1], tiled, y[m0:m1], m1 - m0, N, K, 0)
                return y
            if M <= self.SKINNY_ROWS or out_dtype == torch.float32:
                # few rows (decode), or float32 logits: the weight-streaming MFMA kernel,
                # 64 rows at a time
                wp = tiled
                if wp is None:
                    wp = getattr(matrix, "w", matrix)
                    self._want(wp, "linear matrix")
                for m0 in range(0, M, self.SKINNY_ROWS):
                    m1 = min(M, m0 + self.SKINNY_ROWS)
                    self._call(self.lib.tli_gemm_skinny_bf16, x[m0:m1].data_ptr(), wp.data_ptr(),
                               y[m0:m1].data_ptr(), m1 - m0, N, K, _dtype_code(out_dtype),
                               0 if tiled is None else 1, self.skinny_cfg, self._stream())
                return y
            if tiled is not None and out_dtype == torch.bfloat16 and self._rows_kernel_wins(x, matrix, tiled, M, N, K, 0):
                return self._linear_rows(x, tiled, y, M, N, K, 0, deferred or sums_only)
            # many rows (prefill) where the library was asked for: its matrix product, as the
            # reference uses its library for more than one row (kernels/src/matmul_kernel_cuda.cu:84-91)
            w = getattr(matrix, "w", matrix)
            self._want(w, "linear matrix")
            torch.matmul(x, w.t(), out=y)
            return y
        w = getattr(matrix, "w", matrix)
        self._want(w, "linear matrix")
        self._call(self.lib.tli_gemm_plain, x.data_ptr(), w.data_ptr(), y.data_ptr(), M, N, K,
                   _dtype_code(x.dtype), _dtype_code(w.dtype), _dtype_code(out_dtype), self._stream())
        return y

    def _product_into_residual(self, p: PendingProduct, resid, weight, eps) -> NormedRows:
        """resid += x W^T, and the rows of the norm that follows, its factor still owed."""
        x, m = p.x, p.matrix
        M, K = x.shape
        N = _shape_of(m)[0]
        self._want(x, "linear input", torch.bfloat16, (M, _shape_of(m)[1]))
        if tuple(resid.shape) != (M, N):
            raise KernelError(f"the product gives {(M, N)}, the residual is {tuple(resid.shape)}")
        xw = torch.empty((M, N), dtype=torch.bfloat16, device=self.device)
        ssq = torch.empty(((N + 15) // 16, M), dtype=torch.float32, device=self.device)
        self._call(self.lib.tli_gemm_skinny_fused_bf16, x.data_ptr(), m.tiled.data_ptr(), None, M, N, K, 0,
                   None, 0, 0.0, resid.data_ptr(), weight.data_ptr(), xw.data_ptr(), ssq.data_ptr(), 0,
                   self._stream())
        return NormedRows(xw, ssq, eps)

    def _linear_normed(self, x: NormedRows, m, tiled, gated: int, out_dtype=None):
        """y = normed rows . W^T with the rows' factor applied to the outputs."""
        M, K = x.xw.shape
        if tiled is None:
            raise KernelError("normed rows that still owe their factor need a matrix in the decode layout")
        if out_dtype not in (None, torch.bfloat16):
            raise KernelError("normed rows that still owe their factor give bfloat16 products")
        rows_out = _shape_of(m)[0]
        if _shape_of(m)[1] != K:
            raise KernelError(f"linear: input has {K} columns, the matrix {_shape_of(m)[1]}")
        N = 2 * m.inter if gated else rows_out
        y = torch.empty((M, m.inter if gated else N), dtype=torch.bfloat16, device=self.device)
        self._call(self.lib.tli_gemm_skinny_fused_bf16, x.xw.data_ptr(), tiled.data_ptr(), y.data_ptr(), M, N, K,
                   gated, x.ssq.data_ptr(), x.ssq.shape[0], x.eps, None, None, None, None, 0, self._stream())
        return y

    def _linear_mid(self, x, tiled, y, M, N, K, gated, deferred=False):
        """17..128 rows (without a gate: up to 256): the kernel that shares x through LDS, k cut into
        ranges when the output alone gives too few workgroups.  ``deferred``: the partial sums of the
        ranges are left for the consumer to add, which saves the pass that adds them."""
        splits = self.mid_splits or self.lib.tli_gemm_mid_splits_rows(M, N, K, gated)
        part = None
        if splits > 1:
            part = torch.empty((splits, M, N), dtype=torch.float32, device=self.device)
        leave = deferred and splits > 1 and not gated and y.dtype == torch.bfloat16
        self._call(self.lib.tli_gemm_mid_bf16, x.data_ptr(), tiled.data_ptr(), None if leave else y.data_ptr(),
                   _ptr(part), M, N, K, _dtype_code(y.dtype), gated, splits, self.mid_cfg, self._stream())
        return DeferredSum(part, y.dtype) if leave else y

    def _rows_kernel_wins(self, x, matrix, tiled, M, N, K, gated) -> bool:
        """Whether this product of more than 128 rows goes to gemm_rows (else to the library).
        With ``many_rows`` = "measure": which one is faster changes with the shape by up to 10%
        either way (how well each one's tiles fill the compute units), so both are timed when a
        shape first comes up: three runs each after one to warm up, a few milliseconds, outside
        any graph capture."""
        if max(M, N + 15) * (K + 127) * 2 >= 1 << 32:
            return False                      # gemm_rows keeps 32-bit offsets into its operands
        if self.many_rows != "measure":
            return self.many_rows == "own"
        key = ((M + 127) // 128, N, K, gated)
        won = self.measured.get(key)
        if won is not None:
            return won
        if torch.cuda.is_current_stream_capturing():
            return False                      # (nothing can be timed now; the shape is measured when it next comes up eagerly)
        y = torch.empty((M, N // 2 if gated else N), dtype=torch.bfloat16, device=self.device)
        wide = torch.empty((M, N), dtype=torch.bfloat16, device=self.device) if gated else None
        w = getattr(matrix, "w", matrix)

        def library():
            if gated:
                torch.matmul(x, w.t(), out=wide)
                self.swiglu(wide)
            else:
                torch.matmul(x, w.t(), out=y)

        def own():
            self._linear_rows(x, tiled, y, M, N, K, gated)

        # (in a model the weights of a layer come from memory, not from the last-level cache where a
        # second run would find them: 384 MB are written between the runs)
        if self._cold is None:
            self._cold = torch.empty(96 << 20, dtype=torch.float32, device=self.device)
        times = []
        for fn in (library, own):
            fn()
            total = 0.0
            for _ in range(3):
                self._cold.fill_(0.0)
                start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                start.record()
                fn()
                stop.record()
                stop.synchronize()
                total += start.elapsed_time(stop)
            times.append(total)
        won = times[1] < times[0]
        self.measured[key] = won
        return won

    def _linear_rows(self, x, tiled, y, M, N, K, gated, deferred=False):
        """Any number of rows from the decode layout; k cut into ranges when the output
        alone gives too few workgroups.  ``deferred``: the partial sums of the ranges are
        left for the consumer to add."""
        splits = self.rows_splits or self.lib.tli_gemm_rows_splits(M, N, K)
        part = None
        if splits > 1:
            part = torch.empty((splits, M, N), dtype=torch.float32, device=self.device)
        leave = deferred and splits > 1 and not gated
        self._call(self.lib.tli_gemm_rows_bf16, x.data_ptr(), tiled.data_ptr(), None if leave else y.data_ptr(),
                   _ptr(part), M, N, K, gated, splits, self.rows_cfg, self._stream())
        return DeferredSum(part, y.dtype) if leave else y

    def linear_plain(self, x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None):
        """The plain tiled kernel for any sizes and dtypes: the reference beside the tuned ones."""
        M, K = x.shape
        N = w.shape[0]
        self._want(x, "linear input")
        self._want(w, "linear matrix", x.dtype, (N, K))
        out_dtype = out_dtype or x.dtype
        y = torch.empty((M, N), dtype=out_dtype, device=self.device)
        self._call(self.lib.tli_gemm_plain, x.data_ptr(), w.data_ptr(), y.data_ptr(), M, N, K,
                   _dtype_code(x.dtype), _dtype_code(w.dtype), _dtype_code(out_dtype), self._stream())
        return y

    def linear_swiglu(self, x: torch.Tensor, m) -> torch.Tensor:
        """silu(x gate^T) * (x up^T) for a ``GatedMatrix``.  Few rows: one pass of
        the weight-streaming kernel over the interleaved layout, the activation in
        its epilogue.  Otherwise the stacked product, then the activation."""
        if isinstance(x, NormedRows):
            return self._linear_normed(x, m, getattr(m, "gated", None), 1)
        M, K = x.shape
        gated = getattr(m, "gated", None) if not self.plain_products else None
        if gated is not None and 0 < M <= self.MID_ROWS_TO and x.dtype == torch.bfloat16:
            self._want(x, "linear input", torch.bfloat16, (M, _shape_of(m)[1]))
            y = torch.empty((M, m.inter), dtype=x.dtype, device=self.device)
            if M >= self.MID_ROWS_FROM:
                return self._linear_mid(x, gated, y, M, 2 * m.inter, K, 1)
            self._call(self.lib.tli_gemm_skinny_bf16, x.data_ptr(), gated.data_ptr(), y.data_ptr(), M,
                       2 * m.inter, K, BF16, 2, self.skinny_cfg if self.skinny_cfg >= 20 else 0, self._stream())
            return y
        if (gated is not None and x.dtype == torch.bfloat16 and K % 8 == 0
                and self._rows_kernel_wins(x, m, gated, M, 2 * m.inter, K, 1)):
            self._want(x, "linear input", torch.bfloat16, (M, _shape_of(m)[1]))
            y = torch.empty((M, m.inter), dtype=x.dtype, device=self.device)
            return self._linear_rows(x, gated, y, M, 2 * m.inter, K, 1)
        return self.swiglu(self.linear(x, m))

    def swiglu(self, gu: torch.Tensor) -> torch.Tensor:
        rows, two = gu.shape
        if two % 2:
            raise KernelError("swiglu input must hold gate and up side by side")
        self._want(gu, "swiglu input")
        out = torch.empty((rows, two // 2), dtype=gu.dtype, device=self.device)
        self._call(self.lib.tli_swiglu, gu.data_ptr(), out.data_ptr(), rows, two // 2,
                   _dtype_code(gu.dtype), self._stream())
        return out

    def qkv_to_cache(self, qkv, step, cache, heads, kv_heads, head_dim, q_norm, k_norm, rotary, queries=True):
        """Norms and rotation of q and k, k and v into the cache; returns q.  Without
        ``queries`` only the keys and values are done (bfloat16 heads of 64, 128, 256),
        the values by a kernel of their own that writes runs of slots."""
        T = step.num_rows
        q_dim, kv_dim = heads * head_dim, kv_heads * head_dim
        self._want(qkv, "qkv", None, (T, q_dim + 2 * kv_dim))
        q = torch.empty((T, q_dim), dtype=qkv.dtype, device=self.device) if queries else None
        qw, qe = q_norm if q_norm is not None else (None, 0.0)
        kw, ke = k_norm if k_norm is not None else (None, 0.0)
        for w in (qw, kw):
            if w is not None:
                self._want(w, "head norm weight", torch.float32, (head_dim,))
        cos = sin = None
        rd = npos = 0
        if rotary is not None:
            cos, sin, rd = self._rotary(rotary, step)
            npos = cos.shape[0]
        write = 1 if (cache is not None and cache.writes) else 0
        k_ptr = v_ptr = tab_ptr = None
        width = page = pages = 0
        if write:
            kc, vc = cache.record("k"), cache.record("v")
            g = cache.group
            self._check_cache(kc, vc, g, kv_heads, head_dim, qkv.dtype, step)
            k_ptr, v_ptr, tab_ptr = kc.data_ptr(), vc.data_ptr(), g.tables.data_ptr()
            width, page, pages = g.table_width, g.page_size, kc.shape[0]
        if (not queries and write and qkv.dtype == torch.bfloat16 and head_dim in (64, 128, 256) and page >= 8
                and (rotary is None or rd == head_dim) and not self.separate_cache_writes):
            # keys and values in one pass (prompt portions: the attention kernel takes q from qkv itself)
            self._call(self.lib.tli_keys_values_to_cache, qkv.data_ptr(), k_ptr, v_ptr, step.row_start.data_ptr(),
                       step.seq_start.data_ptr(), step.num_seqs, T, tab_ptr, width, page, pages, heads, kv_heads,
                       head_dim, _ptr(kw), float(ke), _ptr(cos), _ptr(sin), npos, self._stream())
            return None
        self._call(self.lib.tli_qkv_to_cache, qkv.data_ptr(), _ptr(q), k_ptr, v_ptr,
                   step.positions.data_ptr(), step.seq_of_row.data_ptr(), tab_ptr, width, page, pages,
                   T, heads, kv_heads, head_dim, _ptr(qw), float(qe), _ptr(kw), float(ke),
                   _ptr(cos), _ptr(sin), rd, npos, write, 0 if queries else 1, _dtype_code(qkv.dtype),
                   self._stream())
        if write and not queries:
            self._call(self.lib.tli_values_to_cache, qkv.data_ptr(), v_ptr, step.row_start.data_ptr(),
                       step.seq_start.data_ptr(), step.num_seqs, T, tab_ptr, width, page, pages, heads,
                       kv_heads, head_dim, self._stream())
        return q

    def _rotary(self, rotary, step):
        """(cos, sin, rotary_dim) of what a mixer passes as ``rotary``, checked.  The kernels turn
        the pairs (i, i + rotary_dim/2); a fourth element that names another pairing is refused."""
        cos, sin, rd = rotary[0], rotary[1], int(rotary[2])
        if len(rotary) > 3 and rotary[3] != "half":
            raise KernelError(f"the kernels rotate the pairs (i, i + rotary_dim/2) of a head, not the pairing "
                              f"'{rotary[3]}'; the attention part reorders a head's elements for that")
        npos = cos.shape[0]
        self._want(cos, "cos table", torch.float32, (npos, rd // 2))
        self._want(sin, "sin table", torch.float32, (npos, rd // 2))
        if step.max_seq_len > npos:
            raise KernelError(f"a position reaches {step.max_seq_len}, the rotation table has {npos}")
        return cos, sin, rd

    def _check_cache(self, kc, vc, g, kv_heads, head_dim, dtype, step):
        pages = kc.shape[0]
        self._want(kc, "key cache", dtype, (pages, kv_heads, g.page_size, head_dim))
        self._want(vc, "value cache", dtype, (pages, kv_heads, head_dim, g.page_size))
        self._want(g.tables, "block tables", torch.int32, (step.num_seqs, g.table_width))
        if (step.max_seq_len + g.page_size - 1) // g.page_size > g.table_width:
            raise KernelError("a block table is narrower than its sequence needs")

    def paged_attention(self, q, step, cache, heads, kv_heads, head_dim, scale, window):
        T = step.num_rows
        self._want(q, "queries", None, (T, heads * head_dim))
        if cache is None:
            raise KernelError("attention needs a cache layer")
        kc, vc, g = cache.record("k"), cache.record("v"), cache.group
        self._check_cache(kc, vc, g, kv_heads, head_dim, q.dtype, step)
        out = torch.empty_like(q)
        if q.dtype == torch.bfloat16 and head_dim <= 256 and g.page_size >= 4 and not self.force_plain:
            if step.max_rows_per_seq == 1 and g.page_size >= 8:
                return self._attention_decode(q, out, step, kc, vc, g, heads, kv_heads, head_dim, scale, window)
            self._call(self.lib.tli_attention_prefill_bf16, q.data_ptr(), out.data_ptr(), kc.data_ptr(),
                       vc.data_ptr(), step.row_start.data_ptr(), step.seq_start.data_ptr(), step.num_seqs,
                       T, g.tables.data_ptr(), g.table_width, g.page_size, kc.shape[0], heads, kv_heads,
                       head_dim, float(scale), int(window or 0), self._prefill_mode(step, T),
                       self._stream())
            return out
        self._call(self.lib.tli_attention_plain, q.data_ptr(), out.data_ptr(), kc.data_ptr(),
                   vc.data_ptr(), step.positions.data_ptr(), step.seq_of_row.data_ptr(),
                   g.tables.data_ptr(), g.table_width, g.page_size, kc.shape[0], T, heads, kv_heads,
                   head_dim, float(scale), int(window or 0), _dtype_code(q.dtype), self._stream())
        return out

    def qkv_attention(self, qkv, step, cache, heads, kv_heads, head_dim, q_norm, k_norm, rotary, scale, window):
        """From the raw projections to the attention output: norms and rotation of q
        and k, k and v into the cache, attention over the cache.  A decode step (one
        row a sequence) does all of it in the attention kernel where the sizes allow;
        other steps run qkv_to_cache and paged_attention.  ``qkv`` may be a ``DeferredSum``:
        the kernel of a decode step adds the partial sums itself."""
        sums = None
        if isinstance(qkv, DeferredSum):
            sums = qkv
            if not (step.max_rows_per_seq == 1 and qkv.dtype == torch.bfloat16 and cache is not None
                    and head_dim % 64 == 0 and head_dim <= 256 and heads // kv_heads <= 16
                    and cache.group.page_size >= 8 and not self.force_plain and not self.unfused_decode
                     and (rotary is None or rotary[2] == head_dim)):
                qkv, sums = self.resolve(qkv), None
        fusable = (qkv.dtype == torch.bfloat16 and cache is not None and head_dim % 64 == 0
                   and head_dim <= 256 and not self.force_plain and not self.unfused_decode
                   and (rotary is None or rotary[2] == head_dim))
        if (fusable and step.max_rows_per_seq > 1 and head_dim != 192 and cache.group.page_size >= 8
                and self.prefill_direct != 1):
            return self._qkv_attention_prefill(qkv, step, cache, heads, kv_heads, head_dim, q_norm, k_norm,
                                               rotary, scale, window)
        fused = (fusable and step.max_rows_per_seq == 1 and heads // kv_heads <= 16
                 and cache.group.page_size >= 8)
        if not fused:
            q = self.qkv_to_cache(qkv, step, cache, heads, kv_heads, head_dim, q_norm, k_norm, rotary)
            return self.paged_attention(q, step, cache, heads, kv_heads, head_dim, scale, window)
        T = step.num_rows
        if sums is not None:
            self._want(sums.parts, "partial sums of qkv", torch.float32,
                       (sums.parts.shape[0], T, (heads + 2 * kv_heads) * head_dim))
        else:
            self._want(qkv, "qkv", None, (T, (heads + 2 * kv_heads) * head_dim))
        kc, vc, g = cache.record("k"), cache.record("v"), cache.group
        self._check_cache(kc, vc, g, kv_heads, head_dim, qkv.dtype, step)
        qw, qe = q_norm if q_norm is not None else (None, 0.0)
        kw, ke = k_norm if k_norm is not None else (None, 0.0)
        for w in (qw, kw):
            if w is not None:
                self._want(w, "head norm weight", torch.float32, (head_dim,))
        cos = sin = None
        if rotary is not None:
            cos, sin, rd = self._rotary(rotary, step)
        out = torch.empty((T, heads * head_dim), dtype=qkv.dtype, device=self.device)
        splits, per_split, partial = self._decode_splits(step.num_rows, step.reach, g, heads, kv_heads, head_dim, window,
                                                         getattr(step, "skew", 1))
        if splits == 1 and self._a_wave_a_row(T, per_split, g, heads, kv_heads, head_dim):
            splits = 0
        self._call(self.lib.tli_qkv_attention_decode_bf16, None if sums is not None else qkv.data_ptr(),
                   out.data_ptr(), _ptr(partial),
                   kc.data_ptr(), vc.data_ptr(), step.positions.data_ptr(), step.seq_of_row.data_ptr(),
                   g.tables.data_ptr(), g.table_width, g.page_size, kc.shape[0], T, heads, kv_heads,
                   head_dim, _ptr(qw), float(qe), _ptr(kw), float(ke), _ptr(cos), _ptr(sin),
                   1 if cache.writes else 0, float(scale), int(window or 0), splits, per_split,
                   None if sums is None else sums.parts.data_ptr(), 0 if sums is None else sums.parts.shape[0],
                   self._stream())
        return out

    def _qkv_attention_prefill(self, qkv, step, cache, heads, kv_heads, head_dim, q_norm, k_norm, rotary,
                               scale, window):
        """Portions of prompts: keys and values go into the cache in one pass, the
        attention kernel norms and rotates its queries itself (a query is read by
        one wave only, so nothing is done twice and q is never written)."""
        T = step.num_rows
        self.qkv_to_cache(qkv, step, cache, heads, kv_heads, head_dim, q_norm, k_norm, rotary, queries=False)
        kc, vc, g = cache.record("k"), cache.record("v"), cache.group
        self._check_cache(kc, vc, g, kv_heads, head_dim, qkv.dtype, step)
        qw, qe = q_norm if q_norm is not None else (None, 0.0)
        cos, sin = (rotary[0], rotary[1]) if rotary is not None else (None, None)
        out = torch.empty((T, heads * head_dim), dtype=qkv.dtype, device=self.device)
        first = self._rows_for_the_decode_kernel(step, heads, kv_heads)
        if first:
            longest = max(step.h_seq_len[:first])
            kw, ke = k_norm if k_norm is not None else (None, 0.0)
            splits, per_split, partial = self._decode_splits(first, max(128, 1 << (longest - 1).bit_length()), g, heads,
                                                             kv_heads, head_dim, window)
            self._call(self.lib.tli_qkv_attention_decode_bf16, qkv.data_ptr(), out.data_ptr(), _ptr(partial),
                       kc.data_ptr(), vc.data_ptr(), step.positions.data_ptr(), step.seq_of_row.data_ptr(),
                       g.tables.data_ptr(), g.table_width, g.page_size, kc.shape[0], first, heads, kv_heads,
                       head_dim, _ptr(qw), float(qe), _ptr(kw), float(ke), _ptr(cos), _ptr(sin),
                       0, float(scale), int(window or 0), splits, per_split, None, 0, self._stream())
        direct = self._prefill_mode(step, T - first, first)
        self._call(self.lib.tli_qkv_attention_prefill_bf16, qkv.data_ptr(), out.data_ptr(), kc.data_ptr(),
                   vc.data_ptr(), step.row_start.data_ptr() + 4 * first, step.seq_start.data_ptr() + 4 * first,
                   step.num_seqs - first, T - first, g.tables.data_ptr() + 4 * first * g.table_width, g.table_width,
                   g.page_size, kc.shape[0], heads, kv_heads,
                   head_dim, _ptr(qw), float(qe), _ptr(cos), _ptr(sin), float(scale), int(window or 0),
                   direct, self._stream())
        return out

    def _rows_for_the_decode_kernel(self, step, heads, kv_heads) -> int:
        """How many of a mixed step's leading sequences go to the decode kernel.  The sequences that
        decode (one row each) stand first in a step that the scheduler made.  The prefill kernel gives
        each of them workgroups that walk all their keys with one row; where that is slower than a
        second launch (see DECODE_BESIDE_FEW, DECODE_BESIDE_MANY) they go to the decode kernel, which
        splits a row's keys over workgroups (their keys and values are in the cache by then)."""
        first = 0
        starts = step.h_row_start
        while first < step.num_seqs and starts[first + 1] - starts[first] == 1:
            first += 1
        if first == 0 or first == step.num_seqs or heads // kv_heads > 16 or self.prefill_direct:
            return 0
        longest = max(step.h_seq_len[:first])
        beside = max(step.h_seq_len[first:step.num_seqs])
        few, many = self.DECODE_BESIDE_FEW, self.DECODE_BESIDE_MANY
        if (first <= few[0] and longest >= few[1] and longest >= few[2] * beside) or \
                (first >= many[0] and step.num_rows - first <= many[1]):
            return first
        return 0

    def _prefill_mode(self, step, rows, first=0):
        """The mode argument of the prefill attention kernels for the sequences from ``first`` on
        (``rows`` rows in all).  Their launch rule wants to know whether the rows have many keys
        before them, and the lengths themselves are on the device: 13 says that they have (the
        longest of those sequences is a quarter longer than all the rows)."""
        longest = max(step.h_seq_len[first:step.num_seqs]) if step.h_seq_len else step.max_seq_len
        if not self.prefill_direct and longest > rows + rows // 4:
            return 13
        return int(self.prefill_direct)

    def _decode_splits(self, T, reach, g, heads, kv_heads, head_dim, window, skew=1):
        """How the keys of ``T`` rows that decode (``reach``: a power of two that the longest
        of their sequences fits) are split over workgroups: they are when the batch alone
        would leave most of the compute units idle and the rows are long enough for the split
        to pay for its merge.  ``skew``: the longest sequence has at least this many times the
        keys of the average one."""
        reach = reach if not window else min(reach, (window + 31) // 32 * 32 + 32)
        groups = T * kv_heads * ((heads // kv_heads + 15) // 16)
        # A split costs a pass that merges the parts (4 to 5 us) and a workgroup that walks no more than
        # 1,500 keys is done in the time of the shortest split run (13 to 17 us against 17.5), so: no split
        # up to a reach of 2,048 keys; beyond, towards one workgroup a compute unit, half of that for 16
        # (row, kv head) pairs and fewer (more parts than that cost more in the merge than they save in the
        # walk), and splits of at least 1,024 keys, of 4,096 from a quarter of the compute units on (there
        # the workgroups already share the memory's rate between them).  Measured at heads of 128, 1 to 64
        # rows of 600 to 32,768 keys, every power of two of splits: this rule is within 8% of the best
        # everywhere; the one before (256 workgroups, 512 keys) was up to 45% over it at 1,024 keys and 20%
        # over it at 1 and 2 rows of 16,384 keys and more.
        # Sequences of unequal lengths: the workgroups of the short ones are done early, so the step's
        # rows count as that many fewer of the longest one's length (32 rows, one of 4,000 keys and 31 of
        # 300: 40 us unsplit, 30 us in four splits; 16 rows of 64 to 2,304 keys: 24.3 and 22.5 us).  With a
        # window every row walks about as many keys.
        if skew > 1 and not window:
            groups = max(1, groups // skew)
        units = self.DECODE_WORKGROUPS
        splits = 1
        if reach > 2 * self.DECODE_SPLIT_KEYS and groups < units:
            aim = units // 2 if groups <= units // 16 else units
            least = self.DECODE_SPLIT_KEYS if groups <= units // 4 else 4 * self.DECODE_SPLIT_KEYS
            splits = max(1, min((aim + groups - 1) // groups, reach // least, 64))
        # (a split's block table entries are kept in LDS: at most 2046 pages a split)
        splits = max(splits, -(-reach // (2046 * g.page_size // 128 * 128)))
        per_split = ((reach + splits - 1) // splits + 127) // 128 * 128
        splits = (reach + per_split - 1) // per_split
        partial = None
        if splits > 1:
            partial = torch.empty((T * heads * splits * (head_dim + 2),), dtype=torch.float32,
                                  device=self.device)
        return splits, per_split, partial

    def _a_wave_a_row(self, T, keys, g, heads, kv_heads, head_dim) -> bool:
        """Whether a decode step of ``T`` rows that see at most ``keys`` keys each goes to the kernel that
        gives every (row, kv head) one wave to itself: when there are four such pairs for every compute
        unit (a wave on its own waits for every block of its keys, so it takes many waves a SIMD to keep
        the chip busy; then it wins because four waves that share out one row's work and merge their sums
        spend most of their instructions on each other.  Measured at Qwen3-8B sizes, 160 keys a row, a whole
        decode step: 32 rows 3.74 -> 3.93 ms, 64 rows 4.09 -> 4.18, 128 rows 5.38 -> 5.28, 256 rows 10.11 ->
        9.73), and a row's keys lie within the 60 pages whose table entries a wave keeps in its lanes."""
        if self.decode_solo == "never" or head_dim not in (64, 128, 256) or keys > 60 * g.page_size:
            return False
        groups = T * kv_heads * ((heads // kv_heads + 15) // 16)
        return self.decode_solo == "always" or groups >= 4 * self.DECODE_WORKGROUPS

    def _attention_decode(self, q, out, step, kc, vc, g, heads, kv_heads, head_dim, scale, window):
        """One row per sequence."""
        T = step.num_rows
        splits, per_split, partial = self._decode_splits(step.num_rows, step.reach, g, heads, kv_heads, head_dim, window,
                                                         getattr(step, "skew", 1))
        self._call(self.lib.tli_attention_decode_bf16, q.data_ptr(), out.data_ptr(), _ptr(partial),
                   kc.data_ptr(), vc.data_ptr(), step.positions.data_ptr(), step.seq_of_row.data_ptr(),
                   g.tables.data_ptr(), g.table_width, g.page_size, kc.shape[0], T, heads, kv_heads,
                   head_dim, float(scale), int(window or 0), splits, per_split, self._stream())
        return out

    def sample(self, logits: torch.Tensor, temperatures: Optional[torch.Tensor] = None,
               seeds: Optional[torch.Tensor] = None, top_p: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Token ids int32 [rows].  ``temperatures`` float32 [rows] (None: greedy);
        ``seeds`` int64 [rows], one draw seed per row; ``top_p`` float32 [rows] or None."""
        rows, vocab = logits.shape
        self._want(logits, "logits", torch.float32)
        if temperatures is not None:
            self._want(temperatures, "temperatures", torch.float32, (rows,))
            if seeds is None:
                raise KernelError("sampling with a temperature needs seeds")
            self._want(seeds, "seeds", torch.int64, (rows,))
        if top_p is not None:
            self._want(top_p, "top_p", torch.float32, (rows,))
        out = torch.empty((rows,), dtype=torch.int32, device=self.device)
        scratch = torch.empty((self.lib.tli_sample_scratch_bytes(rows),), dtype=torch.uint8, device=self.device)
        self._call(self.lib.tli_sample, logits.data_ptr(), rows, vocab, _ptr(temperatures),
                   _ptr(seeds) if temperatures is not None else None,
                   _ptr(top_p) if temperatures is not None else None, out.data_ptr(), scratch.data_ptr(),
                   self._stream())
        return out


def sample_uniform(seed: int, token: int) -> float:
    """The uniform number the sampling kernel draws for (seed, token)."""
    lib = load_library()
    seed &= (1 << 64) - 1
    return float(lib.tli_sample_uniform(seed & 0xFFFFFFFF, seed >> 32, token))
