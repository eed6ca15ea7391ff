"""The kernels as Python calls on torch tensors.

``load_ops()`` loads the compiled library (building it first if no up-to-date one
exists) and fails loudly when that is impossible: there is no fallback.  Each
method checks what only the Python side can know (device, dtype, contiguity), hands
raw pointers and the current HIP stream to the entry point, and raises
``KernelError`` with the library's message when it refuses its operands.
"""
from __future__ import annotations

import ctypes as C
import threading
from typing import Dict, Optional

import torch

from . import build as _build

XR_F32, XR_BF16 = 0, 1
_CODE = {torch.float32: XR_F32, torch.bfloat16: XR_BF16}
# activations of a gated feed-forward, by the code the kernels know them under (XR_ACT_* of common.h)
GATE_ACTIVATIONS = {"silu": 0}


class KernelError(RuntimeError):
    pass


def activation_code(name: str) -> int:
    try:
        return GATE_ACTIVATIONS[name]
    except KeyError:
        raise KernelError(f"gate activation {name!r} is not built into the kernels (known: {sorted(GATE_ACTIVATIONS)})") from None


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _CODE[dt]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16, not {dt}") from None


_p, _i, _f, _sz, _u32 = C.c_void_p, C.c_int, C.c_float, C.c_size_t, C.c_uint32

_PROTOS = {
    "xr_embedding": [_p, _p, _p, _i, _i, _i, _f, _i, _i, _p],
    "xr_rmsnorm": [_p, _p, _p, _p, _i, _i, _i, _f, _i, _i, _p],
    "xr_rope_kv_write": [_p, _p, _p, _i, _p, _p, _p, _p, _p, _p, _i, _p, _i, _i, _i, _i, _i, _i, _f, _i, _i, _i, _p],
    "xr_gate_mul": [_p, _p, _i, _i, _i, _i, _i, _p],
    "xr_add": [_p, _p, _sz, _i, _p],
    "xr_fill_rows": [_p, _p, _i, _sz, _u32, _p],
    "xr_convert": [_p, _p, _sz, _i, _i, _p],
    "xr_stream_read": [_p, _sz, _p, _i, _p],
    "xr_gemm_ref": [_p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _p],
    "xr_gemm_bf16": [_p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _p, _sz, _p, _p, _p],
    "xr_pack_weight": [_p, _p, _i, _i, _p],
    "xr_rope_table": [_p, _p, _p, _i, _i, _f, _p],
    "xr_attention_ref": [_p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _f, _i, _i, _p],
    "xr_sample": [_p, _p, _i, _i, _i, _p, _p, _p, _p, _p, _p, _p, _p, _i, _p, _i, _p, _p],
}


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


class PackedWeight:
    """A bfloat16 weight matrix ``[rows, cols]`` in the order the MFMA kernels read it: blocks of
    16 rows x 32 columns, 1 KB each (``data[row group, column block, row, column]``), rows and
    columns padded with zeros.  Made by
    ``Ops.pack_weight``; ``Ops.linear`` and ``Ops.linear_gated`` take it in place of the matrix."""

    def __init__(self, data: torch.Tensor, rows: int, cols: int):
        self.data, self.rows, self.cols = data, rows, cols

    @property
    def shape(self):
        return (self.rows, self.cols)

    @property
    def dtype(self):
        return self.data.dtype

    @property
    def device(self):
        return self.data.device


class UnscaledRows:
    """The rows of an RMSNorm that still lack their division by the root mean square:
    ``data [M, E]`` (bfloat16) holds ``x * weight``, ``sumsq [P, 16]`` partial sums of ``x^2`` per
    row (row t's sum is ``sumsq[:, t].sum()``), so the norm's row t is
    ``data[t] * rsqrt(sumsq[:, t].sum() / E + eps)``.  As that factor is one number a row, a
    product ``rows @ w^T`` may apply it to its result instead: ``Ops.linear`` and
    ``Ops.linear_gated`` take this in place of the rows.  Made by ``Ops.linear_add_rmsnorm``."""

    MAX_ROWS = 16

    def __init__(self, data: torch.Tensor, sumsq: torch.Tensor, eps: float):
        self.data, self.sumsq, self.eps = data, sumsq, eps

    @property
    def shape(self):
        return self.data.shape

    @property
    def dtype(self):
        return self.data.dtype

    @property
    def device(self):
        return self.data.device


class _GemmNorm(C.Structure):
    """XrGemmNorm of the library."""
    _fields_ = [("ss_in", _p), ("n_ss", _i), ("ss_inv_width", _f), ("ss_eps", _f), ("norm_w", _p),
                ("norm_w_bf16", _i), ("xg", _p), ("ss_out", _p), ("ss_out_rows", _i)]


class _GemmRope(C.Structure):
    """XrGemmRope of the library."""
    _fields_ = [("positions", _p), ("req_of_token", _p), ("block_table", _p), ("table_stride", _i),
                ("inv_freq", _p), ("H", _i), ("Hk", _i), ("D", _i), ("rot", _i), ("interleaved", _i),
                ("mscale", _f), ("page_size", _i), ("q_out", _p), ("k_cache", _p), ("v_cache", _p), ("cs_table", _p)]


def paired_order(D: int, rot: int) -> list:
    """``order[c]`` = the channel of a head that stands at column ``c`` in "paired order": a
    rotation's pairs ``(j, j + rot/2)`` side by side in groups of 16 columns (8 first halves, then
    their 8 partners), channels from ``rot`` on in place.  ``rot`` must be a multiple of 16."""
    if rot % 16 or rot > D:
        raise ValueError(f"paired order needs a rotary width that is a multiple of 16 and at most {D}, got {rot}")
    order = list(range(D))
    half = rot // 2
    for d in range(rot):
        hi, j = (1, d - half) if d >= half else (0, d)
        order[(j // 8) * 16 + hi * 8 + j % 8] = d
    return order


class _Lib:
    def __init__(self, path: str, protos: Dict[str, list]):
        self.path = path
        self.dll = C.CDLL(path)
        self.dll.xr_last_error.restype = C.c_char_p
        self.dll.xr_last_error.argtypes = []
        for name, args in protos.items():
            fn = getattr(self.dll, name)
            fn.argtypes = args
            fn.restype = C.c_int
            setattr(self, name, fn)

    def check(self, rc: int) -> None:
        if rc != 0:
            raise KernelError(self.dll.xr_last_error().decode("utf-8", "replace"))


class Ops:
    """All kernels of the forward pass and of sampling."""

    def __init__(self, lib: _Lib):
        self.lib = lib
        self._attn_libs: Dict[int, object] = {}
        self.use_mfma = True
        self.fold_norms = True      # False: linear_add_rmsnorm always runs the norm's own kernel
        self.fuse_rope = True       # False: project_rope_kv_write always runs two kernels
        self.ROPE_TILE_ROWS = int(lib.dll.xr_rope_tile_rows())
        self.FINISH_ROWS = self.ROPE_TILE_ROWS - 1

    # -- checks -----------------------------------------------------------------
    @staticmethod
    def _dev(*ts: Optional[torch.Tensor]) -> None:
        for t in ts:
            if t is not None and not t.is_cuda:
                raise KernelError("kernel operand is not on the GPU (there is no CPU path)")

    @staticmethod
    def _contig(t: torch.Tensor, what: str) -> None:
        if not t.is_contiguous():
            raise KernelError(f"{what} must be contiguous")

    # -- element-wise and row-wise ----------------------------------------------
    def embedding(self, table, ids: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
        """``out[t] = table[ids[t]] * scale`` as 32-bit rows; ``table`` is a matrix or a ``PackedWeight``."""
        packed = isinstance(table, PackedWeight)
        data = table.data if packed else table
        self._dev(data, ids)
        self._contig(data, "embedding table")
        T, (V, E) = ids.numel(), table.shape
        out = torch.empty((T, E), dtype=torch.float32, device=data.device)
        self.lib.check(self.lib.xr_embedding(out.data_ptr(), data.data_ptr(), ids.data_ptr(), T, E, V,
                                             float(scale), dtype_code(data.dtype), 1 if packed else 0, _stream()))
        return out

    def rmsnorm(self, x: torch.Tensor, w: Optional[torch.Tensor], eps: float, out_dtype: torch.dtype,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """RMSNorm of the rows of 32-bit ``x`` (or of the rows ``rows`` selects)."""
        self._dev(x, w, rows)
        if x.dtype != torch.float32 or x.dim() != 2 or x.stride(1) != 1:
            raise KernelError("rmsnorm input must be float32 [rows, width] with unit column stride")
        E = x.shape[1]
        if w is not None and (w.numel() != E or not w.is_contiguous()):
            raise KernelError(f"rmsnorm weight has {w.numel()} elements, the row has {E}")
        R = x.shape[0] if rows is None else rows.numel()
        out = torch.empty((R, E), dtype=out_dtype, device=x.device)
        self.lib.check(self.lib.xr_rmsnorm(out.data_ptr(), x.data_ptr(), _ptr(w), _ptr(rows), R, E, x.stride(0),
                                           float(eps), dtype_code(out_dtype),
                                           dtype_code(w.dtype) if w is not None else XR_F32, _stream()))
        return out

    def gate_mul(self, gu: torch.Tensor, activation: str = "silu") -> torch.Tensor:
        """``act(gu[:, :F]) * gu[:, F:]``."""
        self._dev(gu)
        T, F2 = gu.shape
        F = F2 // 2
        if gu.stride(1) != 1 or F2 % 2:
            raise KernelError("gate_mul input must be [rows, 2F] with unit column stride")
        out = torch.empty((T, F), dtype=gu.dtype, device=gu.device)
        self.lib.check(self.lib.xr_gate_mul(out.data_ptr(), gu.data_ptr(), T, F, gu.stride(0),
                                            dtype_code(gu.dtype), activation_code(activation), _stream()))
        return out

    def silu_mul(self, gu: torch.Tensor) -> torch.Tensor:
        """``silu(gu[:, :F]) * gu[:, F:]``."""
        return self.gate_mul(gu, "silu")

    def add_(self, x: torch.Tensor, y: torch.Tensor) -> None:
        """``x += y`` with 32-bit ``x``."""
        self._dev(x, y)
        if x.dtype != torch.float32 or x.shape != y.shape:
            raise KernelError(f"add_: x must be float32 and shapes equal, got {x.dtype} {tuple(x.shape)} {tuple(y.shape)}")
        self._contig(x, "add_ x")
        self._contig(y, "add_ y")
        self.lib.check(self.lib.xr_add(x.data_ptr(), y.data_ptr(), x.numel(), dtype_code(y.dtype), _stream()))

    def fill_rows_(self, base: torch.Tensor, rows: Optional[torch.Tensor], n_rows: int, value_bits: int = 0) -> None:
        """Set whole rows of ``base`` (first axis) to a 32-bit pattern."""
        self._dev(base, rows)
        self._contig(base, "fill_rows_ base")
        row_bytes = base[0].numel() * base.element_size()
        if row_bytes % 4:
            raise KernelError("fill_rows_: a row must be a multiple of 4 bytes")
        self.lib.check(self.lib.xr_fill_rows(base.data_ptr(), _ptr(rows), int(n_rows), row_bytes // 4,
                                             value_bits & 0xFFFFFFFF, _stream()))

    def convert(self, x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
        self._dev(x)
        self._contig(x, "convert input")
        out = torch.empty(x.shape, dtype=dtype, device=x.device)
        self.lib.check(self.lib.xr_convert(out.data_ptr(), x.data_ptr(), x.numel(), dtype_code(x.dtype),
                                           dtype_code(dtype), _stream()))
        return out

    def stream_read(self, buf: torch.Tensor, blocks: int = 2048) -> torch.Tensor:
        """Read ``buf`` once, every workgroup a range of its own (the yardstick for what a kernel
        that only reads gets from memory); returns ``[blocks]`` int32 whose XOR is the XOR of the
        buffer's 32-bit words."""
        self._dev(buf)
        self._contig(buf, "stream_read buffer")
        sink = torch.empty((blocks,), dtype=torch.int32, device=buf.device)
        self.lib.check(self.lib.xr_stream_read(buf.data_ptr(), buf.numel() * buf.element_size(), sink.data_ptr(),
                                               blocks, _stream()))
        return sink

    # -- matrix product ---------------------------------------------------------
    GEMM_WORKSPACE_BYTES = 96 << 20
    ROPE_TILE_ROWS = 512    # from here the q/k/v product has tiles enough with K whole, and its tile kernel rotates and caches
    FINISH_ROWS = 511       # up to here the kernel that adds a product's K ranges up rotates and caches (the library's own number)

    def _gemm_workspace(self, device):
        """Room for the sums of K ranges when a product with few rows is split (one buffer per process;
        products on one stream use it one after another)."""
        ws = getattr(self, "_gemm_ws", None)
        if ws is None or ws.device != device:
            ws = torch.empty((self.GEMM_WORKSPACE_BYTES // 4,), dtype=torch.float32, device=device)
            self._gemm_ws = ws
        return ws.data_ptr(), self.GEMM_WORKSPACE_BYTES

    def _mfma_ok(self, a: torch.Tensor, w: torch.Tensor) -> bool:
        return (self.use_mfma and a.dtype == torch.bfloat16 and a.shape[1] % 8 == 0 and a.stride(0) % 8 == 0
                and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)

    def pack_weight(self, w: torch.Tensor, gated: bool = False):
        """``w`` for use as the weight of ``linear`` (``gated``: of ``linear_gated``): packed for
        the MFMA kernels where they will serve it (bfloat16, a width that is a multiple of 8, for
        gate and up rows a height that is a multiple of 32), else ``w`` itself."""
        if not (self.use_mfma and w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[1] % 8 == 0):
            return w
        N, K = w.shape
        if gated and N % 32:
            return w
        self._dev(w)
        self._contig(w, "pack_weight input")
        data = torch.empty((-(-N // 16), -(-K // 32), 16, 32), dtype=torch.bfloat16, device=w.device)
        self.lib.check(self.lib.xr_pack_weight(data.data_ptr(), w.data_ptr(), N, K, _stream()))
        return PackedWeight(data, N, K)

    def linear(self, a: torch.Tensor, w, bias: Optional[torch.Tensor] = None,
               out_dtype: Optional[torch.dtype] = None, out: Optional[torch.Tensor] = None,
               accumulate: bool = False, variant: int = 0, _then: Optional[_GemmNorm] = None) -> torch.Tensor:
        """``a [M, K] @ w [N, K]^T (+ bias)``; with ``accumulate`` added into 32-bit ``out``.

        bfloat16 operands run on the matrix cores (32-bit accumulation); float32 operands, and
        shapes the MFMA kernels do not take, run the plain 32-bit FMA kernel.  ``w`` is a matrix
        or a ``PackedWeight``.
        """
        packed = isinstance(w, PackedWeight)
        wt = w.data if packed else w
        norm, a = self._norm_before(a, _then)
        self._dev(a, wt, bias, out)
        if a.dim() != 2 or len(w.shape) != 2 or a.shape[1] != w.shape[1]:
            raise KernelError(f"linear: shapes {tuple(a.shape)} x {tuple(w.shape)}^T do not fit")
        if a.dtype != w.dtype:
            raise KernelError(f"linear: input is {a.dtype}, weight is {w.dtype}")
        if a.stride(1) != 1:
            raise KernelError("linear: input must have unit column stride")
        self._contig(wt, "linear weight")
        M, K = a.shape
        N = w.shape[0]
        if out is None:
            if accumulate:
                raise KernelError("linear: accumulate needs an output")
            out = torch.empty((M, N), dtype=out_dtype or a.dtype, device=a.device)
        elif out.shape != (M, N) or out.stride(1) != 1:
            raise KernelError(f"linear: output is {tuple(out.shape)}, product is {(M, N)}")
        if bias is not None and (bias.dtype != torch.float32 or bias.numel() != N):
            raise KernelError("linear: bias must be float32 [N]")
        if self._mfma_ok(a, wt):
            self.lib.check(self.lib.xr_gemm_bf16(out.data_ptr(), a.data_ptr(), wt.data_ptr(), _ptr(bias), M, N, K,
                                                 a.stride(0), out.stride(0), dtype_code(out.dtype),
                                                 1 if accumulate else 0, 0, variant, 1 if packed else 0,
                                                 *self._gemm_workspace(a.device),
                                                 C.addressof(norm) if norm is not None else None, None, _stream()))
            return out
        if norm is not None:
            raise KernelError("linear: rows that still lack their norm's scale need the MFMA kernels")
        if packed:
            raise KernelError("linear: a packed weight needs bfloat16 rows that are 16-byte aligned")
        self.lib.check(self.lib.xr_gemm_ref(out.data_ptr(), a.data_ptr(), w.data_ptr(), _ptr(bias), M, N, K,
                                            a.stride(0), out.stride(0), dtype_code(a.dtype),
                                            dtype_code(out.dtype), 1 if accumulate else 0, _stream()))
        return out

    @staticmethod
    def _norm_before(a, then: Optional[_GemmNorm]):
        """(what the library needs to know about a norm folded into this product, the rows)"""
        if not isinstance(a, UnscaledRows):
            return then, a
        if a.data.shape[0] > UnscaledRows.MAX_ROWS:
            raise KernelError(f"a product takes at most {UnscaledRows.MAX_ROWS} rows that still lack their norm's scale")
        norm = then if then is not None else _GemmNorm()
        norm.ss_in, norm.n_ss = a.sumsq.data_ptr(), a.sumsq.shape[0]
        norm.ss_inv_width, norm.ss_eps = 1.0 / a.data.shape[1], float(a.eps)
        return norm, a.data

    def linear_add_rmsnorm(self, a, w, residual: torch.Tensor, norm_weight: Optional[torch.Tensor], eps: float,
                           out_dtype: torch.dtype, bias: Optional[torch.Tensor] = None, defer: bool = False):
        """``residual += a @ w^T (+ bias)``, then the RMSNorm of the updated rows.

        With ``defer`` the caller says that what reads the result is a ``linear`` or
        ``linear_gated``: for at most 16 bfloat16 rows the product's kernel then also writes the
        weighted rows and their partial sums of squares, and an ``UnscaledRows`` comes back, whose
        scale the next product applies.  With more rows, where the product is split over K (always
        from 17 to 64 rows, above that when its tiles are too few for the chip), the kernel that adds up
        the K ranges takes whole rows and writes the finished norm.  In every other case the norm's own
        kernel runs.  A tensor comes back in both."""
        wt = w.data if isinstance(w, PackedWeight) else w
        rows = a.data if isinstance(a, UnscaledRows) else a
        M, N = rows.shape[0], w.shape[0]
        fits = (self.fold_norms and out_dtype == torch.bfloat16 and norm_weight is not None
                and N % 8 == 0 and norm_weight.numel() == N and norm_weight.is_contiguous()
                and residual.dtype == torch.float32 and self._mfma_ok(rows, wt))
        deferred = fits and defer and M <= UnscaledRows.MAX_ROWS
        # More rows: where the product is split over K (always from 17 to 64 rows, above that when
        # its tiles are too few for the chip), the kernel that adds the parts up takes whole rows and
        # writes the finished norm; the library says whether it did.
        whole = fits and M > UnscaledRows.MAX_ROWS and N % 4 == 0 and residual.stride(0) % 4 == 0
        if deferred or whole:
            self._dev(norm_weight)
            then = _GemmNorm()
            xg = torch.empty((M, N), dtype=torch.bfloat16, device=rows.device)
            parts = -(-N // 16)
            sumsq = torch.empty((parts, 16), dtype=torch.float32, device=rows.device) if deferred else None
            then.norm_w, then.norm_w_bf16 = norm_weight.data_ptr(), dtype_code(norm_weight.dtype)
            then.xg, then.ss_out, then.ss_out_rows = xg.data_ptr(), _ptr(sumsq), parts
            then.ss_inv_width, then.ss_eps = 1.0 / N, float(eps)
            self.linear(a, w, bias=bias, out=residual, accumulate=True, _then=then)
            if then.ss_out_rows < 0:
                return xg                                   # the finished norm
            if deferred:
                return UnscaledRows(xg, sumsq[:then.ss_out_rows], eps)
            return self.rmsnorm(residual, norm_weight, eps, out_dtype)      # the library declined
        self.linear(a, w, bias=bias, out=residual, accumulate=True)
        return self.rmsnorm(residual, norm_weight, eps, out_dtype)

    def linear_gated(self, a: torch.Tensor, w, bias: Optional[torch.Tensor] = None, activation: str = "silu",
                     variant: int = 0) -> torch.Tensor:
        """``act(a @ w[:F]^T) * (a @ w[F:]^T)`` for ``w [2F, K]`` = gate rows then up rows
        (a matrix, or a ``PackedWeight`` made with ``gated=True``); ``activation`` is one of
        ``GATE_ACTIVATIONS``."""
        act = activation_code(activation)
        packed = isinstance(w, PackedWeight)
        wt = w.data if packed else w
        norm, a = self._norm_before(a, None)
        F = w.shape[0] // 2
        if w.shape[0] % 2:
            raise KernelError("linear_gated: the weight must have an even number of rows")
        if self._mfma_ok(a, wt):
            self._dev(a, wt, bias)
            self._contig(wt, "linear_gated weight")
            M, K = a.shape
            if K != w.shape[1] or a.stride(1) != 1:
                raise KernelError(f"linear_gated: shapes {tuple(a.shape)} x {tuple(w.shape)}^T do not fit")
            if bias is not None and (bias.dtype != torch.float32 or bias.numel() != 2 * F):
                raise KernelError("linear_gated: bias must be float32 [2F]")
            out = torch.empty((M, F), dtype=a.dtype, device=a.device)
            self.lib.check(self.lib.xr_gemm_bf16(out.data_ptr(), a.data_ptr(), wt.data_ptr(), _ptr(bias), M, F, K,
                                                 a.stride(0), F, dtype_code(out.dtype), 2, act, variant,
                                                 1 if packed else 0, *self._gemm_workspace(a.device),
                                                 C.addressof(norm) if norm is not None else None, None, _stream()))
            return out
        if norm is not None:
            raise KernelError("linear_gated: rows that still lack their norm's scale need the MFMA kernels")
        if packed:
            raise KernelError("linear_gated: a packed weight needs bfloat16 rows that are 16-byte aligned")
        return self.gate_mul(self.linear(a, w, bias=bias), activation)

    def linear_swiglu(self, a: torch.Tensor, w, bias: Optional[torch.Tensor] = None, variant: int = 0) -> torch.Tensor:
        """``linear_gated`` with the SiLU gate."""
        return self.linear_gated(a, w, bias=bias, activation="silu", variant=variant)

    # -- attention --------------------------------------------------------------
    def rope_kv_write(self, q_in, k_in, v_in, q_out, k_cache, v_cache, positions, req_of_token,
                      block_table, inv_freq, H: int, Hk: int, D: int, rot: int, interleaved: bool,
                      mscale: float, page_size: int, paired: bool = False) -> None:
        """Rotate queries (into ``q_out``) and keys, and write keys and values to their pages.

        ``q_in``/``k_in``/``v_in`` are 32-bit views with one common row stride.  ``paired``: the
        channels of every query and key head come in ``paired_order``.
        """
        self._dev(q_in, k_in, v_in, q_out, k_cache, v_cache, positions, req_of_token, block_table, inv_freq)
        T = positions.numel()
        ins = [t for t in (q_in, k_in, v_in) if t is not None]
        if any(t.dtype != torch.float32 or t.stride(-1) != 1 for t in ins):
            raise KernelError("rope_kv_write: inputs must be float32 with unit column stride")
        strides = {t.stride(0) for t in ins}
        if len(strides) > 1:
            raise KernelError("rope_kv_write: q, k and v inputs must share a row stride")
        stride = strides.pop() if strides else 0
        store = q_out if q_out is not None else k_cache
        if k_cache is not None and q_out is not None and k_cache.dtype != q_out.dtype:
            raise KernelError("rope_kv_write: query output and cache differ in dtype")
        self.lib.check(self.lib.xr_rope_kv_write(
            _ptr(q_in), _ptr(k_in), _ptr(v_in), stride, _ptr(q_out), _ptr(k_cache), _ptr(v_cache),
            positions.data_ptr(), _ptr(req_of_token), _ptr(block_table),
            block_table.stride(0) if block_table is not None else 0, _ptr(inv_freq), T, H, Hk, D, rot,
            1 if interleaved else 0, float(mscale), page_size, dtype_code(store.dtype), 1 if paired else 0,
            _stream()))

    def rope_table(self, positions: torch.Tensor, inv_freq: torch.Tensor, mscale: float = 1.0) -> torch.Tensor:
        """``[T, rot/2, 2]`` float32: cosine and sine (times ``mscale``) of every row's angles, as
        ``project_rope_kv_write`` takes them for a product of many rows (``cs_table``); the same for
        every layer that rotates by ``inv_freq``, so a step needs it once."""
        self._dev(positions, inv_freq)
        T, half = positions.numel(), inv_freq.numel()
        out = torch.empty((T, half, 2), dtype=torch.float32, device=positions.device)
        self.lib.check(self.lib.xr_rope_table(out.data_ptr(), positions.data_ptr(), inv_freq.data_ptr(), T, half,
                                              float(mscale), _stream()))
        return out

    def project_rope_kv_write(self, h, w, bias, k_cache, v_cache, positions, req_of_token, block_table,
                              inv_freq, H: int, Hk: int, D: int, rot: int, interleaved: bool, mscale: float,
                              page_size: int, paired: bool = False, cs_table=None, variant: int = 0) -> torch.Tensor:
        """``[q | k | v] = h @ w^T (+ bias)``, queries and keys rotated, keys and values written
        to their pages; returns the rotated queries ``[T, H*D]`` in the compute dtype.

        ``w`` holds ``H`` query heads, then ``Hk`` key heads and ``Hk`` value heads (``Hk`` = 0 and
        no caches: queries alone); with ``paired`` its query and key rows are in ``paired_order``.
        Up to 16 bfloat16 rows (``h`` may be an ``UnscaledRows``) the product's kernel rotates and
        stores its own result, up to 511 the kernel that adds the product's K ranges up does, from
        512 the tile kernel (with the rows' cosines and sines from a table made first), which
        saves a kernel; in float32, and where the kernels' conditions on sizes do not hold, the
        product and ``rope_kv_write`` run one after the other.  ``cs_table``: a callable that returns the
        step's ``rope_table`` (asked for only where the tile kernel rotates).  ``variant``: a tile kernel
        by number instead of the library's choice (tests; from 512 rows on)."""
        rows = h.data if isinstance(h, UnscaledRows) else h
        wt = w.data if isinstance(w, PackedWeight) else w
        T, Q, KV = rows.shape[0], H * D, Hk * D
        if w.shape[0] != Q + 2 * KV:
            raise KernelError(f"projection has {w.shape[0]} rows, {H} query and 2 x {Hk} key/value heads of {D} need {Q + 2 * KV}")
        q = torch.empty((T, Q), dtype=rows.dtype, device=rows.device)
        if (self.fuse_rope and (T <= self.FINISH_ROWS or T >= self.ROPE_TILE_ROWS) and self._mfma_ok(rows, wt) and D % 16 == 0
                and (T * w.shape[0] * 4 if T <= self.FINISH_ROWS else T * (rot // 2 + 1) * 8) <= self.GEMM_WORKSPACE_BYTES
                and (Hk == 0 or (k_cache.dtype == torch.bfloat16 and v_cache.dtype == torch.bfloat16))
                and (rot == 0 or interleaved or (paired and rot % 16 == 0))):
            self._dev(rows, wt, bias, k_cache, v_cache, positions, req_of_token, block_table, inv_freq)
            self._contig(wt, "projection weight")
            if rows.shape[1] != w.shape[1] or rows.stride(1) != 1:
                raise KernelError(f"projection: shapes {tuple(rows.shape)} x {tuple(w.shape)}^T do not fit")
            if bias is not None and (bias.dtype != torch.float32 or bias.numel() != w.shape[0]):
                raise KernelError("projection: bias must be float32 [N]")
            norm, rows = self._norm_before(h, None)
            rp = _GemmRope()
            rp.positions, rp.req_of_token, rp.block_table = positions.data_ptr(), _ptr(req_of_token), _ptr(block_table)
            rp.table_stride = block_table.stride(0) if block_table is not None else 0
            rp.inv_freq, rp.H, rp.Hk, rp.D, rp.rot = _ptr(inv_freq), H, Hk, D, rot
            rp.interleaved, rp.mscale, rp.page_size = 1 if interleaved else 0, float(mscale), page_size
            rp.q_out, rp.k_cache, rp.v_cache = q.data_ptr(), _ptr(k_cache) if Hk else None, _ptr(v_cache) if Hk else None
            table = cs_table() if (cs_table is not None and T >= self.ROPE_TILE_ROWS and rot > 0) else None
            rp.cs_table = _ptr(table)
            self.lib.check(self.lib.xr_gemm_bf16(None, rows.data_ptr(), wt.data_ptr(), _ptr(bias), T, w.shape[0],
                                                 rows.shape[1], rows.stride(0), w.shape[0], XR_F32, 0, 0, variant,
                                                 1 if isinstance(w, PackedWeight) else 0,
                                                 *self._gemm_workspace(rows.device),
                                                 C.addressof(norm) if norm is not None else None,
                                                 C.addressof(rp), _stream()))
            return q
        proj = self.linear(h, w, bias=bias, out_dtype=torch.float32)
        k_in = proj[:, Q:Q + KV] if Hk else None
        v_in = proj[:, Q + KV:Q + 2 * KV] if Hk else None
        self.rope_kv_write(proj[:, :Q], k_in, v_in, q, k_cache if Hk else None, v_cache if Hk else None, positions,
                           req_of_token, block_table, inv_freq, H, Hk, D, rot, interleaved, mscale, page_size,
                           paired=paired)
        return q

    def attention(self, q, k_cache, v_cache, ctx, group: int, H: int, Hk: int, D: int, page_size: int,
                  scale: float, window: Optional[int] = None) -> torch.Tensor:
        """Causal attention of every token of the step over its request's cached keys and values.

        bfloat16 runs on the matrix cores (head sizes in steps of 16 up to 256, pages of at least
        16 positions); float32, and what the MFMA kernel does not take, runs the 32-bit kernel.
        """
        positions, req_of_token, block_table = ctx.positions, ctx.req_of_token, ctx.block_table(group)
        self._dev(q, k_cache, v_cache, positions, req_of_token, block_table)
        T = positions.numel()
        self._contig(q, "attention queries")
        if q.dtype != k_cache.dtype or q.dtype != v_cache.dtype:
            raise KernelError("attention: queries and cache differ in dtype")
        if H % Hk:
            raise KernelError(f"attention: {H} query heads are not a multiple of {Hk} key/value heads")
        out = torch.empty((T, H * D), dtype=q.dtype, device=q.device)
        if self.use_mfma and q.dtype == torch.bfloat16 and D % 16 == 0 and 16 <= D <= 256 and page_size >= 16:
            lib = self.attention_lib(D)
            plan = ctx.attention_plan(group, H // Hk, window, Hk, page_size)
            part_o = part_ml = None
            if plan.n_slots:
                part_o = torch.empty((plan.n_slots, Hk, 32, D), dtype=torch.float32, device=q.device)
                part_ml = torch.empty((plan.n_slots, Hk, 32, 2), dtype=torch.float32, device=q.device)
            lib.check(lib.xr_attention_mfma(
                out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), plan.items.data_ptr(),
                plan.n_items, plan.n_cta_items, _ptr(plan.jobs), plan.n_jobs, ctx.cu_q.data_ptr(),
                ctx.starts_dev.data_ptr(), block_table.data_ptr(), block_table.stride(0), _ptr(part_o), _ptr(part_ml), H, Hk, D, page_size,
                float(scale), int(window or 0), _stream()))
            return out
        self.lib.check(self.lib.xr_attention_ref(
            out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), positions.data_ptr(),
            req_of_token.data_ptr(), block_table.data_ptr(), block_table.stride(0), T, H, Hk, D, page_size,
            float(scale), int(window or 0), dtype_code(q.dtype), _stream()))
        return out

    def attention_lib(self, D: int) -> "_Lib":
        """The MFMA attention library for head size ``D`` (compiled at first use)."""
        lib = self._attn_libs.get(D)
        if lib is None:
            unit = f"attn_d{D}"
            path = _build.find_built(unit) or _build.build_unit(unit)
            lib = _Lib(path, {"xr_attention_mfma": [_p, _p, _p, _p, _p, _i, _i, _p, _i, _p, _p, _p, _i, _p, _p,
                                                    _i, _i, _i, _i, _f, _i, _p]})
            self._attn_libs[D] = lib
        return lib

    # -- sampling ---------------------------------------------------------------
    def sample(self, logits, temp, draw, top_k=None, top_p=None, min_p=None, repeat_penalty=None,
               recent=None, n_recent=None, exempt=None) -> torch.Tensor:
        """One token id per row of 32-bit ``logits`` (rows with a penalty are changed in place)."""
        self._dev(logits, temp, draw, top_k, top_p, min_p, repeat_penalty, recent, n_recent, exempt)
        if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
            raise KernelError("sample: logits must be float32 [rows, vocab]")
        W, V = logits.shape
        out = torch.empty((W,), dtype=torch.int32, device=logits.device)
        # room for the greedy rows' first pass (32 ranges a row) when a row is long enough to need one
        greedy_ws = torch.empty((W, 32, 2), dtype=torch.float32, device=logits.device) if V >= 8192 else None
        self.lib.check(self.lib.xr_sample(
            out.data_ptr(), logits.data_ptr(), W, V, logits.stride(0), temp.data_ptr(), _ptr(top_k),
            _ptr(top_p), _ptr(min_p), _ptr(repeat_penalty), draw.data_ptr(), _ptr(recent), _ptr(n_recent),
            recent.shape[1] if recent is not None else 0, _ptr(exempt),
            exempt.numel() if exempt is not None else 0, _ptr(greedy_ws), _stream()))
        return out


_LOCK = threading.Lock()
_OPS: Optional[Ops] = None


def load_ops() -> Ops:
    """The kernel library, loaded once per process (compiled first if it must be)."""
    global _OPS
    with _LOCK:
        if _OPS is None:
            path = _build.find_built("kernels") or _build.build_unit("kernels")
            _OPS = Ops(_Lib(path, _PROTOS))
        return _OPS
