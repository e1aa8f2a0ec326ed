"""The hand-written gfx950 kernels, bound through ctypes.

`HipKernels` is the only compute backend of the library.  Every method checks
on the host what its kernel and grid assume (dtype, device, contiguity, sizes),
then launches on the current HIP stream.  There is no fallback: if the shared
library cannot be built or loaded, constructing `HipKernels` raises.

Tensors are torch tensors used as typed device buffers; no torch operator runs
here.
"""
from __future__ import annotations

import ctypes
from ctypes import c_double, c_float, c_int, c_longlong, c_void_p
from typing import Optional

import torch

from .. import build as _build
from .dry import query

F32, BF16 = 0, 1
ABI_VERSION = 10  # lq_abi_version() of the library these wrappers were written for
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}


class KernelLibraryError(RuntimeError):
    """The kernel library is missing, or a kernel refused its arguments."""


_LIB = None


def load_library() -> ctypes.CDLL:
    global _LIB
    if _LIB is not None:
        return _LIB
    try:
        path = _build.ensure_built()
    except Exception as e:  # BuildError, OSError
        raise KernelLibraryError(
            f"the gfx950 kernel library could not be built: {e}\n"
            "This library has no CPU or library fallback; it needs hipcc (ROCm) to compile its kernels."
        ) from e
    try:
        lib = ctypes.CDLL(path)
    except OSError as e:
        raise KernelLibraryError(f"cannot load {path}: {e}") from e
    lib.lq_last_error.restype = ctypes.c_char_p
    lib.lq_abi_version.restype = c_int
    if lib.lq_abi_version() != ABI_VERSION:
        raise KernelLibraryError(f"{path} speaks version {lib.lq_abi_version()} of the kernel interface, "
                                 f"this package version {ABI_VERSION}: build it again")
    # The entry points that a prompt step calls most take plain Python numbers (declared argument types
    # save making a ctypes object for each of them: a call from Python is 5 us instead of 10, where the
    # launch itself is 3).
    vp, ci, cl, cf = c_void_p, c_int, c_longlong, c_float
    lib.lq_linear.argtypes = [vp, vp, vp, ci, ci, ci, ci, ci, ci, ci, ci, ci, cl, ci, ci, vp]
    lib.lq_linear_swiglu.argtypes = [vp, vp, vp, ci, ci, ci, ci, ci, ci, ci, ci, ci, vp]
    lib.lq_rmsnorm.argtypes = [vp, vp, ci, ci, cl, vp, cf, vp, ci, ci, ci, vp]
    lib.lq_attention.argtypes = [vp, ci, vp, ci, ci, ci, ci, ci, ci, ci, vp, vp, vp, vp, vp, ci, vp, vp, ci, cf, ci, ci, ci,
                                 vp, cl, vp, cl, vp, vp, ci, ci, vp, ci, ci, cl, ci, vp]
    lib.lq_rope_store_pieces.argtypes = [vp, ci, ci, cl, vp, ci, ci, ci, ci, ci, vp, vp, vp, vp, vp, ci, vp, vp, ci, vp]
    _LIB = lib
    return lib


def _ptr(t: Optional[torch.Tensor]) -> c_void_p:
    return c_void_p(0 if t is None else t.data_ptr())


ptr = _ptr  # for parts that launch a kernel of their own through `HipKernels.call`


def _code(t: torch.Tensor) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise KernelLibraryError(f"unsupported tensor dtype {t.dtype}") from None


class PackedWeight:
    """A weight [N, K] whose memory is in the packed order of `HipKernels.pack_weight`: what the products and
    the embedding take in a tensor's place.  It answers what they ask of a weight (shape, dtype, strides of the
    matrix it stands for, the address) and is no tensor: nothing else can read it by mistake."""

    packed = True

    def __init__(self, data: torch.Tensor, rows: int, cols: int) -> None:
        self.data, self.shape, self.dtype, self.device = data, torch.Size((rows, cols)), data.dtype, data.device
        self.is_cuda = data.is_cuda

    def data_ptr(self) -> int:
        return self.data.data_ptr()

    def dim(self) -> int:
        return 2

    def stride(self, i: Optional[int] = None):
        st = (self.shape[1], 1)
        return st if i is None else st[i]

    def is_contiguous(self) -> bool:
        return True

    def contiguous(self) -> "PackedWeight":
        return self

    def numel(self) -> int:
        return self.data.numel()

    def element_size(self) -> int:
        return self.data.element_size()


def _packed(w) -> int:
    return 1 if getattr(w, "packed", False) else 0


class HipKernels:
    name = "hip-gfx950"

    def __init__(self) -> None:
        self.lib = load_library()
        if not torch.cuda.is_available():
            raise KernelLibraryError("no HIP device is visible; this library runs on a gfx950 GPU only")
        self._stream: Optional[int] = None
        self.force_generic = False  # route linear and attention to the size-agnostic kernels
        self.pack_weights = True    # `pack_weight` packs what may be packed (False: it hands every weight back)
        # ticket counters of the decoding attention (one for each row and kv head of a launch); a launch
        # finds them zero and leaves them zero, so launches through one object must not overlap
        self._tickets: dict = {}  # device -> the counters

    def prepare(self, device: torch.device) -> None:
        """What an engine asks once before its first step on `device`: everything that this object allocates
        by itself is there afterwards, so that no launch under a stream capture has to allocate."""
        self.tickets(device)

    def tickets(self, device: torch.device) -> torch.Tensor:
        """The ticket counters on `device` (made at the first launch there, or by `prepare`)."""
        device = torch.device(device)
        if device.index is None:
            device = torch.device(device.type, torch.cuda.current_device())
        t = self._tickets.get(device)
        if t is None:
            t = self._tickets[device] = torch.zeros(1 << 18, dtype=torch.int32, device=device)
        return t

    # ------------------------------------------------------------------ plumbing
    def use_stream(self, stream: Optional["torch.cuda.Stream"]) -> None:
        """Launch on `stream` from now on (None: ask torch for its current stream each call)."""
        self._stream = None if stream is None else int(stream.cuda_stream)

    @property
    def stream(self) -> c_void_p:
        if self._stream is not None:
            return c_void_p(self._stream)
        return c_void_p(int(torch.cuda.current_stream().cuda_stream))

    def _check(self, rc: int) -> None:
        if rc != 0:
            raise KernelLibraryError(self.lib.lq_last_error().decode("utf-8", "replace"))

    def call(self, symbol: str, *args) -> None:
        """Launches an `extern "C" int symbol(..., hipStream_t)` of the library on this object's stream: for a
        part that brings a kernel of its own (a `.hip` file beside the others is compiled into the library; the
        function checks its arguments with LQ_REQUIRE and returns non-zero after `lq_set_error`).  `args` are
        ctypes values; `ptr(tensor)` gives a tensor's address."""
        fn = getattr(self.lib, symbol, None)
        if fn is None:
            raise KernelLibraryError(f"the kernel library has no function {symbol}")
        self._check(fn(*args, self.stream))

    @staticmethod
    def _dev(*tensors: Optional[torch.Tensor]) -> None:
        for t in tensors:
            if t is None:
                continue
            if not t.is_cuda:
                raise KernelLibraryError("kernel arguments must live on the GPU")
            if t.dim() > 0 and t.stride(-1) != 1 and t.shape[-1] != 1:
                raise KernelLibraryError("kernel arguments must be contiguous in their last dimension")

    @staticmethod
    def _mat(t: torch.Tensor, what: str):
        """(rows, columns, row stride in elements) of a 2-D tensor on the GPU whose rows are dense: `_dev` and
        `_rows2d` in one pass."""
        sh = t.shape
        if len(sh) != 2:
            raise KernelLibraryError(f"{what}: expected a 2-D tensor, found shape {tuple(sh)}")
        if not t.is_cuda:
            raise KernelLibraryError("kernel arguments must live on the GPU")
        st = t.stride()
        if st[1] != 1 and sh[1] != 1:
            raise KernelLibraryError("kernel arguments must be contiguous in their last dimension")
        return sh[0], sh[1], (st[0] if sh[0] > 1 else max(st[0], sh[1]))

    @staticmethod
    def _rows2d(t: torch.Tensor, what: str) -> int:
        """Row stride in elements of a 2-D view whose last dimension is dense."""
        if t.dim() != 2:
            raise KernelLibraryError(f"{what}: expected a 2-D tensor, found shape {tuple(t.shape)}")
        return int(t.stride(0)) if t.shape[0] > 1 else max(int(t.stride(0)), int(t.shape[1]))

    @staticmethod
    def _i32(t: torch.Tensor, what: str, n: int) -> None:
        if t.dtype != torch.int32 or not t.is_contiguous() or t.numel() < n:
            raise KernelLibraryError(f"{what}: need a contiguous int32 tensor of at least {n} entries")

    # ------------------------------------------------------------------ kernels
    def pack_weight(self, w: torch.Tensor):
        """The weight [N, K] of a product as the products like to read it, made once when weights are bound:
        a `PackedWeight` (8 rows' slabs of 64 k side by side, so that the slab of a tile of rows is one run of
        memory instead of 128 bytes from every row) where every kernel that can meet a weight of this size reads
        that order (bfloat16, wide, K in 64s), else w itself.  `linear`, `linear_swiglu`, `linear_residual`,
        `linear_scaled` and `embed` take either."""
        if not self.pack_weights or getattr(w, "packed", False) or w.dim() != 2 or w.dtype not in _DTYPE_CODE \
                or not w.is_cuda or not w.is_contiguous():
            return w
        n, k = w.shape
        if not self.lib.lq_weight_packable(c_int(_DTYPE_CODE[w.dtype]), c_int(n), c_int(k)):
            return w
        out = torch.empty_like(w)
        self._check(self.lib.lq_pack_weight(_ptr(w), _ptr(out), c_int(n), c_int(k), self.stream))
        return PackedWeight(out, n, k)

    def embed(self, table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> None:
        """out[r, :] = scale * float32(table[tokens[r], :]); zeros where tokens[r] is no row of the table"""
        self._dev(table, tokens, out)
        rows, width = out.shape
        self._i32(tokens, "embed tokens", rows)
        if out.dtype != torch.float32 or not out.is_contiguous() or not table.is_contiguous():
            raise KernelLibraryError("embed: out must be dense float32, the table dense")
        if table.dim() != 2 or table.shape[1] != width:
            raise KernelLibraryError(f"embed: table {tuple(table.shape)} does not match width {width}")
        self._check(self.lib.lq_embed(_ptr(table), c_int(_code(table)), _ptr(tokens), _ptr(out),
                                      c_int(rows), c_int(width), c_int(table.shape[0]), c_int(_packed(table)),
                                      c_float(scale), self.stream))

    @staticmethod
    def _pieces(delta: Optional[torch.Tensor], like: torch.Tensor, what: str):
        """A delta is shaped like x, or holds several pieces [pieces, rows, width] whose sum is meant
        (`linear_pieces`).  -> (pieces, elements between pieces)"""
        if delta is None:
            return 0, 0
        if not delta.is_contiguous() or tuple(delta.shape[-2:]) != tuple(like.shape) or delta.dim() not in (2, 3):
            raise KernelLibraryError(f"{what}: delta must be dense and shaped like x, or a stack of such pieces")
        return (delta.shape[0], like.numel()) if delta.dim() == 3 else (1, 0)

    def rmsnorm(self, x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
                delta: Optional[torch.Tensor] = None) -> None:
        """(x += delta;) out = x / sqrt(mean(x^2) + eps) * weight, row by row; x is float32."""
        rows, width, ldx = self._mat(x, "rmsnorm: x")
        if delta is not None:
            self._dev(delta)
        pieces, stride = self._pieces(delta, x, "rmsnorm")
        if x.dtype != torch.float32 or (ldx != width and rows > 1):
            raise KernelLibraryError("rmsnorm: x must be dense float32")
        if weight.dtype != torch.float32 or weight.numel() != width or not weight.is_contiguous() or not weight.is_cuda:
            raise KernelLibraryError(f"rmsnorm: weight must be float32 of {width} entries")
        ro, wo, ldo = self._mat(out, "rmsnorm: out")
        if ro != rows or wo != width or (ldo != width and rows > 1):
            raise KernelLibraryError("rmsnorm: out must be dense and shaped like x")
        rc = self.lib.lq_rmsnorm(x.data_ptr(), 0 if delta is None else delta.data_ptr(),
                                 _code(delta) if delta is not None else 0, pieces, stride, weight.data_ptr(),
                                 float(eps), out.data_ptr(), _code(out), rows, width, self.stream)
        if rc:
            self._check(rc)

    def add(self, x: torch.Tensor, delta: torch.Tensor) -> None:
        """x += delta (x float32)."""
        self._dev(x, delta)
        if x.dtype != torch.float32 or not x.is_contiguous():
            raise KernelLibraryError("add: x must be dense float32")
        pieces, _ = self._pieces(delta, x, "add")
        for piece in (delta if pieces > 1 or delta.dim() == 3 else (delta,)):
            self._check(self.lib.lq_add(_ptr(x), _ptr(piece), c_int(_code(piece)), c_longlong(x.numel()),
                                        self.stream))

    def cast(self, src: torch.Tensor, out: torch.Tensor) -> None:
        self._dev(src, out)
        if src.shape != out.shape or not src.is_contiguous() or not out.is_contiguous():
            raise KernelLibraryError("cast: dense tensors of one shape are needed")
        self._check(self.lib.lq_cast(_ptr(src), c_int(_code(src)), _ptr(out), c_int(_code(out)),
                                     c_longlong(src.numel()), self.stream))

    @query
    def linear_pieces(self, dtype: torch.dtype, m: int, n: int, k: int) -> int:
        """In how many pieces `linear` would like to leave this product (1: whole).  A caller whose
        consumer adds pieces (`rmsnorm`, `add`, `gather_rows` with a stacked delta) may pass an output
        [pieces, M, N]; the kernel then splits K over more blocks and each piece is a partial sum."""
        if dtype not in _DTYPE_CODE:
            return 1
        return int(self.lib.lq_linear_splits(c_int(_DTYPE_CODE[dtype]), c_int(m), c_int(n), c_int(k),
                                             c_int(1 if self.force_generic else 0)))

    def linear(self, x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> None:
        """out[M, N] = x[M, K] . w[N, K]^T with 32-bit accumulation; or out[pieces, M, N] with
        `linear_pieces` pieces that sum to it."""
        m, k, ldx = self._mat(x, "linear: x")
        n, kw, ldw = self._mat(w, "linear: w")
        pieces, stride = 1, 0
        if out.dim() == 3:
            pieces, stride = out.shape[0], m * n
            if not out.is_cuda or not out.is_contiguous() or pieces != self.linear_pieces(x.dtype, m, n, k):
                raise KernelLibraryError(f"linear: {pieces} pieces asked (dense, on the GPU), linear_pieces says "
                                         f"{self.linear_pieces(x.dtype, m, n, k)}")
            mo, no, ldc = out.shape[1], out.shape[2], n
        else:
            mo, no, ldc = self._mat(out, "linear: out")
        if kw != k or mo != m or no != n:
            raise KernelLibraryError(
                f"linear: x {tuple(x.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} do not fit")
        if x.dtype != w.dtype:
            raise KernelLibraryError(f"linear: x is {x.dtype} but w is {w.dtype}")
        rc = self.lib.lq_linear(x.data_ptr(), w.data_ptr(), out.data_ptr(), _code(x), _code(out), m, n, k, ldx, ldw,
                                ldc, pieces, stride, 1 if self.force_generic else 0, _packed(w), self.stream)
        if rc:
            self._check(rc)

    # -- the two products around a norm, for a few rows (decoding): x += act . w^T leaves every row's
    # sum of squares in parts, and the product after the norm normalises its input from them itself
    @query
    def linear_fused_parts(self, dtype: torch.dtype, m: int, n: int, k: int) -> int:
        """How many parts `linear_residual` leaves a row for [m, k] x [n, k]^T; 0: these kernels do
        not take the size (use `linear` and `rmsnorm`)."""
        if self.force_generic or dtype not in _DTYPE_CODE:
            return 0
        return int(self.lib.lq_linear_fused_parts(c_int(_DTYPE_CODE[dtype]), c_int(m), c_int(n), c_int(k)))

    def linear_residual(self, act: torch.Tensor, w: torch.Tensor, x: torch.Tensor, sq_parts: torch.Tensor,
                        gain: Optional[torch.Tensor] = None, scaled: Optional[torch.Tensor] = None) -> None:
        """x[M, N] (float32, in place) += act[M, K] . w[N, K]^T; sq_parts[M, parts] (float32) takes, a part
        per block of columns, the sums of squares of the updated rows; with gain [N] (float32),
        scaled[M, N] takes (x * gain) in the dtype of act: the input of `linear_scaled`."""
        self._dev(act, w, x, sq_parts, gain, scaled)
        m, k = act.shape
        n = w.shape[0]
        if w.shape[1] != k or tuple(x.shape) != (m, n) or act.dtype != w.dtype:
            raise KernelLibraryError(f"linear_residual: act {tuple(act.shape)}, w {tuple(w.shape)}, x {tuple(x.shape)} do not fit")
        if x.dtype != torch.float32 or sq_parts.dtype != torch.float32 or sq_parts.dim() != 2 \
                or sq_parts.shape[0] != m or not sq_parts.is_contiguous():
            raise KernelLibraryError("linear_residual: x and sq_parts [M, parts] must be float32")
        if (gain is None) != (scaled is None):
            raise KernelLibraryError("linear_residual: gain and scaled come together")
        if gain is not None and (gain.dtype != torch.float32 or gain.numel() != n or not gain.is_contiguous()
                                 or tuple(scaled.shape) != (m, n) or scaled.dtype != act.dtype):
            raise KernelLibraryError("linear_residual: gain must be float32 [N], scaled [M, N] in the dtype of act")
        self._check(self.lib.lq_linear_residual(_ptr(act), _ptr(w), _ptr(x), _ptr(sq_parts), _ptr(gain), _ptr(scaled),
                                                c_int(self._rows2d(scaled, "scaled") if scaled is not None else 0),
                                                c_int(_code(act)), c_int(m), c_int(n), c_int(k),
                                                c_int(self._rows2d(act, "act")), c_int(self._rows2d(w, "w")),
                                                c_int(self._rows2d(x, "x")), c_int(sq_parts.shape[1]),
                                                c_int(_packed(w)), self.stream))

    def linear_scaled(self, h: torch.Tensor, sq_parts: torch.Tensor, eps: float, w: torch.Tensor,
                      out: torch.Tensor, swiglu: bool = False) -> None:
        """out[r] = (h[r] . w^T) / sqrt(mean + eps), mean being the sum of sq_parts[r, :] over K: with
        h = x * gain this is rmsnorm(x) . w^T.  With `swiglu`, w holds interleaved gate and up rows and
        out is [M, N / 2] (as `linear_swiglu`)."""
        self._dev(h, sq_parts, w, out)
        m, k = h.shape
        n = w.shape[0]
        n_out = n // 2 if swiglu else n
        if w.shape[1] != k or tuple(out.shape) != (m, n_out) or h.dtype != w.dtype:
            raise KernelLibraryError(f"linear_scaled: h {tuple(h.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} do not fit")
        if sq_parts.dtype != torch.float32 or sq_parts.dim() != 2 or sq_parts.shape[0] != m or not sq_parts.is_contiguous():
            raise KernelLibraryError("linear_scaled: sq_parts [M, parts] must be float32")
        self._check(self.lib.lq_linear_scaled(_ptr(h), c_int(self._rows2d(h, "h")), _ptr(sq_parts),
                                              c_int(sq_parts.shape[1]), c_float(eps), _ptr(w), _ptr(out),
                                              c_int(_code(w)), c_int(_code(out)), c_int(m), c_int(n), c_int(k),
                                              c_int(self._rows2d(w, "w")), c_int(self._rows2d(out, "out")),
                                              c_int(1 if swiglu else 0), c_int(_packed(w)), self.stream))

    @query
    def linear_swiglu_supported(self, dtype: torch.dtype, rows_out: int, k: int) -> bool:
        """Whether `linear_swiglu` takes weights of this dtype with `rows_out` (= 2 I) rows and width k."""
        if self.force_generic or dtype not in _DTYPE_CODE:
            return False
        return bool(self.lib.lq_linear_swiglu_supported(c_int(_DTYPE_CODE[dtype]), c_int(rows_out), c_int(k)))

    def linear_swiglu(self, x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> None:
        """out[M, I] = silu(gate) * up with [gate | up] = x . w^T, in one kernel.  w [2 I, K] holds the
        gate and up rows interleaved in groups of 8: rows 16j..16j+7 gate 8j..8j+7, rows 16j+8..16j+15
        up 8j..8j+7 (see `interleave_gate_up`)."""
        m, k, ldx = self._mat(x, "linear_swiglu: x")
        n, kw, ldw = self._mat(w, "linear_swiglu: w")
        mo, no, ldc = self._mat(out, "linear_swiglu: out")
        if kw != k or mo != m or no != n // 2 or n % 16 != 0 or x.dtype != w.dtype:
            raise KernelLibraryError(
                f"linear_swiglu: x {tuple(x.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} do not fit")
        rc = self.lib.lq_linear_swiglu(x.data_ptr(), w.data_ptr(), out.data_ptr(), _code(x), _code(out), m, n, k,
                                       ldx, ldw, ldc, _packed(w), self.stream)
        if rc:
            self._check(rc)

    @staticmethod
    def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
        """The weight layout `linear_swiglu` reads (done once, when weights are bound)."""
        inner, width = gate.shape
        return torch.stack([gate.view(inner // 8, 8, width), up.view(inner // 8, 8, width)], dim=1) \
            .reshape(2 * inner, width).contiguous()

    def swiglu(self, gate_up: torch.Tensor, out: torch.Tensor) -> None:
        """out[r, i] = silu(gate_up[r, i]) * gate_up[r, I + i]"""
        self._dev(gate_up, out)
        rows, width = out.shape
        if tuple(gate_up.shape) != (rows, 2 * width) or not gate_up.is_contiguous() or not out.is_contiguous():
            raise KernelLibraryError("swiglu: gate_up must be dense [rows, 2 I] and out dense [rows, I]")
        self._check(self.lib.lq_swiglu(_ptr(gate_up), c_int(_code(gate_up)), _ptr(out), c_int(_code(out)),
                                       c_int(rows), c_int(width), self.stream))

    def gather_rows(self, x: torch.Tensor, rows: torch.Tensor, out: torch.Tensor,
                    delta: Optional[torch.Tensor] = None) -> None:
        """out[i, :] = x[rows[i], :] (+ delta[rows[i], :])"""
        self._dev(x, rows, out, delta)
        n, width = out.shape
        self._i32(rows, "gather rows", n)
        pieces, stride = self._pieces(delta, x, "gather_rows")
        if x.dtype != torch.float32 or out.dtype != torch.float32 or x.shape[1] != width:
            raise KernelLibraryError("gather_rows: float32 tensors of one width are needed")
        if not x.is_contiguous() or not out.is_contiguous():
            raise KernelLibraryError("gather_rows: dense tensors are needed")
        self._check(self.lib.lq_gather_rows(_ptr(x), _ptr(delta), c_int(_code(delta) if delta is not None else 0),
                                            c_int(pieces), c_longlong(stride),
                                            _ptr(rows), _ptr(out), c_int(n), c_int(width), self.stream))

    @query
    def rope_store_takes_table(self, rows: int) -> bool:
        """Whether a step of so many rows is worth a table of cos and sin for `rope_store`: the kernel that
        reads it takes eight positions a workgroup and pays from about a thousand rows on (19 against 22 us at
        2 048 rows and 49 against 74 at 8 192, but 8.7 against 7.1 us at 128 rows)."""
        return rows >= 1024

    @query
    def rope_store_adds_pieces(self, dtype: torch.dtype, rows: int, heads: int, kv_heads: int, head_dim: int) -> bool:
        """Whether `rope_store_pieces` takes q, k and v of such a step as the float32 pieces of a product
        that shares K over blocks (`linear_pieces`): bfloat16 steps of fewer rows than `rope_store` wants a
        table for, head sizes in steps of 16."""
        return (not self.force_generic and dtype == torch.bfloat16 and head_dim % 16 == 0
                and not self.rope_store_takes_table(rows))

    def rope_store_pieces(self, qkv: torch.Tensor, q_out: torch.Tensor, heads: int, kv_heads: int, head_dim: int,
                          freqs: torch.Tensor, row_pos: torch.Tensor, row_seq: torch.Tensor, seq_slot: torch.Tensor,
                          block_table: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, block_size: int) -> None:
        """`rope_store` for qkv float32 [pieces, rows, (heads + 2 kv_heads) * head_dim], the partial sums of
        the projection with q, k and v side by side: adds the pieces in ascending order, rounds the sums to
        bfloat16 as the whole product would have, rotates q (into q_out, bfloat16 [rows, heads * head_dim])
        and k, and writes k and v into the paged cache."""
        self._dev(qkv, q_out, freqs, row_pos, row_seq, seq_slot, block_table, kcache, vcache)
        if qkv.dim() != 3 or qkv.dtype != torch.float32 or not qkv.is_contiguous() \
                or qkv.shape[2] != (heads + 2 * kv_heads) * head_dim:
            raise KernelLibraryError("rope_store_pieces: qkv must be dense float32 [pieces, rows, (heads + 2 kv_heads) * head_dim]")
        pieces, rows, width = qkv.shape
        if q_out.dtype != torch.bfloat16 or tuple(q_out.shape) != (rows, heads * head_dim) \
                or kcache.dtype != torch.bfloat16 or vcache.dtype != torch.bfloat16:
            raise KernelLibraryError("rope_store_pieces: q_out bfloat16 [rows, heads * head_dim], bfloat16 caches")
        self._i32(row_pos, "row_pos", rows)
        self._i32(row_seq, "row_seq", rows)
        if freqs.dtype != torch.float64 or freqs.numel() != head_dim // 2 or not freqs.is_contiguous():
            raise KernelLibraryError(f"rope_store_pieces: freqs must be float64 of {head_dim // 2} entries")
        if seq_slot.dtype != torch.int32 or block_table.dtype != torch.int32 or block_table.dim() != 2:
            raise KernelLibraryError("rope_store_pieces: seq_slot and block_table must be int32 (table 2-D)")
        nb = kcache.shape[0]
        if tuple(kcache.shape) != (nb, kv_heads, block_size, head_dim) or \
                tuple(vcache.shape) != (nb, kv_heads, head_dim, block_size) or \
                not kcache.is_contiguous() or not vcache.is_contiguous():
            raise KernelLibraryError("rope_store_pieces: cache tensors do not have the paged layout")
        rc = self.lib.lq_rope_store_pieces(
            qkv.data_ptr(), width, pieces, qkv.stride(0), q_out.data_ptr(), self._rows2d(q_out, "q_out"), rows, heads,
            kv_heads, head_dim, freqs.data_ptr(), row_pos.data_ptr(), row_seq.data_ptr(), seq_slot.data_ptr(),
            block_table.data_ptr(), int(block_table.stride(0)), kcache.data_ptr(), vcache.data_ptr(), block_size,
            self.stream)
        if rc:
            self._check(rc)

    def rope_store(self, q: torch.Tensor, k: Optional[torch.Tensor], v: Optional[torch.Tensor],
                   heads: int, kv_heads: int, head_dim: int, freqs: Optional[torch.Tensor],
                   row_pos: torch.Tensor, row_seq: Optional[torch.Tensor] = None,
                   seq_slot: Optional[torch.Tensor] = None, block_table: Optional[torch.Tensor] = None,
                   kcache: Optional[torch.Tensor] = None, vcache: Optional[torch.Tensor] = None,
                   block_size: int = 0, cos_sin: Optional[torch.Tensor] = None,
                   cu_rows: Optional[torch.Tensor] = None) -> None:
        """Rotate q (in place) and k by the rows' positions; write rotated k and v into the paged cache.

        q [rows, >= heads*head_dim], k and v [rows, >= kv_heads*head_dim] (views into one buffer are
        fine); freqs float64 [head_dim/2] or None for no rotation; without a cache only q is rotated.
        With the step's table of cos and sin (`rope_table`: float32 [rows, head_dim/2, 2]) and `cu_rows`
        (the rows lie sequence by sequence, positions consecutive within each) a bfloat16 step that stores
        takes the kernel that works on eight positions at a time; the results are the same bits.
        """
        self._dev(q, k, v, freqs, row_pos, row_seq, seq_slot, block_table, kcache, vcache)
        rows = q.shape[0]
        store = kcache is not None
        self._i32(row_pos, "row_pos", rows)
        if q.shape[1] < heads * head_dim:
            raise KernelLibraryError("rope_store: q is narrower than heads * head_dim")
        if freqs is not None and (freqs.dtype != torch.float64 or freqs.numel() != head_dim // 2
                                  or not freqs.is_contiguous()):
            raise KernelLibraryError(f"rope_store: freqs must be float64 of {head_dim // 2} entries")
        bt_stride = 1
        if store:
            if k is None or v is None or vcache is None or row_seq is None or seq_slot is None or block_table is None:
                raise KernelLibraryError("rope_store: storing needs k, v, both caches and the batch's tables")
            if k.dtype != q.dtype or v.dtype != q.dtype or kcache.dtype != q.dtype or vcache.dtype != q.dtype:
                raise KernelLibraryError("rope_store: q, k, v and the caches must share one dtype")
            if k.shape[0] != rows or v.shape[0] != rows or k.shape[1] < kv_heads * head_dim or v.shape[1] < kv_heads * head_dim:
                raise KernelLibraryError("rope_store: k / v do not match the rows or kv width")
            self._i32(row_seq, "row_seq", rows)
            if seq_slot.dtype != torch.int32 or block_table.dtype != torch.int32 or block_table.dim() != 2:
                raise KernelLibraryError("rope_store: seq_slot and block_table must be int32 (table 2-D)")
            nb = kcache.shape[0]
            if tuple(kcache.shape) != (nb, kv_heads, block_size, head_dim) or \
                    tuple(vcache.shape) != (nb, kv_heads, head_dim, block_size) or \
                    not kcache.is_contiguous() or not vcache.is_contiguous():
                raise KernelLibraryError("rope_store: cache tensors do not have the paged layout")
            bt_stride = int(block_table.stride(0))
        if (store and cos_sin is not None and cu_rows is not None and freqs is not None and q.dtype == torch.bfloat16
                and head_dim % 16 == 0 and block_size % 8 == 0):
            ldq, ldk, ldv = self._rows2d(q, "q"), self._rows2d(k, "k"), self._rows2d(v, "v")
            aligned = ldq % 8 == 0 and ldk % 8 == 0 and all(t.data_ptr() % 16 == 0 for t in (q, k, kcache, vcache, cos_sin))
            if aligned:
                self._dev(cos_sin, cu_rows)
                if cos_sin.dtype != torch.float32 or tuple(cos_sin.shape) != (rows, head_dim // 2, 2) \
                        or not cos_sin.is_contiguous():
                    raise KernelLibraryError("rope_store: cos_sin must be dense float32 [rows, head_dim/2, 2]")
                if cu_rows.dtype != torch.int32 or cu_rows.numel() < 2:
                    raise KernelLibraryError("rope_store: cu_rows must be int32 with an entry past the last sequence")
                self._check(self.lib.lq_rope_store_groups(
                    _ptr(q), _ptr(k), _ptr(v), c_int(rows), c_int(ldq), c_int(ldk), c_int(ldv), c_int(heads),
                    c_int(kv_heads), c_int(head_dim), _ptr(cos_sin), _ptr(row_pos), _ptr(cu_rows),
                    c_int(cu_rows.numel() - 1), _ptr(seq_slot), _ptr(block_table), c_int(bt_stride), _ptr(kcache),
                    _ptr(vcache), c_int(block_size), self.stream))
                return
        self._check(self.lib.lq_rope_store(
            _ptr(q), _ptr(k), _ptr(v), c_int(_code(q)), c_int(rows),
            c_int(self._rows2d(q, "q")), c_int(self._rows2d(k, "k") if k is not None else 0),
            c_int(self._rows2d(v, "v") if v is not None else 0),
            c_int(heads), c_int(kv_heads if store else 0), c_int(head_dim), _ptr(freqs),
            _ptr(row_pos), _ptr(row_seq), _ptr(seq_slot), _ptr(block_table), c_int(bt_stride),
            _ptr(kcache), _ptr(vcache), c_int(block_size), c_int(1 if store else 0), self.stream))

    @query
    def attention_workspace(self, dtype: torch.dtype, rows: int, heads: int, kv_heads: int, head_dim: int,
                            block_size: int, decode: bool, max_len: int) -> int:
        """Float32 entries of scratch that `attention` wants for this launch (0: none)."""
        self.lib.lq_attention_workspace.restype = c_longlong
        if self.force_generic or dtype not in _DTYPE_CODE:
            return 0
        return int(self.lib.lq_attention_workspace(c_int(_DTYPE_CODE[dtype]), c_int(rows), c_int(heads),
                                                   c_int(kv_heads), c_int(head_dim), c_int(block_size),
                                                   c_int(1 if decode else 0), c_int(max_len)))

    @query
    def attention_folds_rope(self, dtype: torch.dtype, heads: int, kv_heads: int, head_dim: int, block_size: int) -> bool:
        """Whether a decoding `attention` launch can rotate q and k and write the cache itself."""
        if self.force_generic or dtype not in _DTYPE_CODE:
            return False
        return bool(self.lib.lq_attention_folds_rope(c_int(_DTYPE_CODE[dtype]), c_int(heads), c_int(kv_heads),
                                                     c_int(head_dim), c_int(block_size)))

    @query
    def attention_on_matrix_cores(self, dtype: torch.dtype, heads: int, kv_heads: int, head_dim: int, block_size: int) -> bool:
        """Whether `attention` runs this shape on its matrix-core kernel, prompts and single tokens alike (keys and
        values of one size, dense rows)."""
        if self.force_generic or dtype not in _DTYPE_CODE:
            return False
        return bool(self.lib.lq_attention_on_matrix_cores(c_int(_DTYPE_CODE[dtype]), c_int(heads), c_int(kv_heads),
                                                          c_int(head_dim), c_int(block_size)))

    @query
    def attention_adds_pieces(self, dtype: torch.dtype, heads: int, kv_heads: int, head_dim: int, block_size: int) -> bool:
        """Whether such a launch also takes q, k and v as the float32 pieces that `linear` leaves where it
        shares K over blocks (`linear_pieces` > 1), and adds them up itself."""
        return self.attention_folds_rope(dtype, heads, kv_heads, head_dim, block_size)

    @query
    def decode_length_bound(self, longest: int) -> int:
        """The bound of the lengths that a decoding `attention` launch shapes its grid by when the longest
        sequence holds `longest` tokens: launches with one bound sum in one order, so a step kept for replay
        serves until a sequence outgrows its bound."""
        bucket = int(self.lib.lq_attention_length_bucket())
        return (max(1, int(longest)) + bucket - 1) // bucket * bucket

    @query
    def decode_lengths_uneven(self, lengths) -> bool:
        """Whether a decoding step with these lengths should tell `attention` that they differ much
        (`uneven`): the kernel library's own rule."""
        n = len(lengths)
        return bool(self.lib.lq_attention_lengths_uneven((c_int * max(1, n))(*[int(x) for x in lengths]), c_int(n)))

    def rope_table(self, freqs: torch.Tensor, row_pos: torch.Tensor, out: torch.Tensor) -> None:
        """out[r, i] = (cos, sin) of row_pos[r] * freqs[i]; float32 [rows, pairs, 2]."""
        self._dev(freqs, row_pos, out)
        rows, half = out.shape[0], out.shape[1]
        self._i32(row_pos, "row_pos", rows)
        if freqs.dtype != torch.float64 or freqs.numel() != half or out.dtype != torch.float32 \
                or tuple(out.shape) != (rows, half, 2) or not out.is_contiguous():
            raise KernelLibraryError("rope_table: freqs float64 [pairs], out dense float32 [rows, pairs, 2]")
        self._check(self.lib.lq_rope_table(_ptr(freqs), _ptr(row_pos), _ptr(out), c_int(rows), c_int(half), self.stream))

    def attention(self, q: torch.Tensor, out: torch.Tensor, heads: int, kv_heads: int, head_dim: int,
                  row_pos: torch.Tensor, row_seq: torch.Tensor, seq_slot: torch.Tensor, cu_rows: torch.Tensor,
                  block_table: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor,
                  block_size: int, scale: float, window: int = 0, decode: bool = False, max_len: int = 0,
                  workspace: Optional[torch.Tensor] = None, k_new: Optional[torch.Tensor] = None,
                  v_new: Optional[torch.Tensor] = None, cos_sin: Optional[torch.Tensor] = None,
                  uneven: bool = False, pieces: int = 1, piece_stride: int = 0) -> None:
        """Causal grouped-query attention of the step's rows over their slots' cached keys.

        `decode` promises one row per sequence; `max_len` is then an upper bound of the lengths
        after this step and `workspace` float32 scratch of `attention_workspace(...)` entries.
        `uneven` says that the sequences of a decoding step differ much in length (the step's
        context knows): the launch then shares the keys out over its workgroups by the true lengths.
        With `cos_sin` (a `rope_table` of this step; only where `attention_folds_rope` says so) q, k_new
        and v_new are the unrotated projections: the launch rotates q and k and writes k and v into
        the cache itself.  With `pieces` > 1 (such a launch only, where `attention_adds_pieces` says so)
        q, k_new and v_new are float32 views into the first of that many partial sums of the projection,
        `piece_stride` elements apart (what `linear` leaves in a 3-D out): the launch adds them up."""
        self._dev(q, out, row_pos, row_seq, seq_slot, cu_rows, block_table, kcache, vcache, workspace)
        rows = q.shape[0]
        batch = seq_slot.numel()
        self._i32(row_pos, "row_pos", rows)
        self._i32(row_seq, "row_seq", rows)
        self._i32(cu_rows, "cu_rows", batch + 1)
        if out.shape[0] != rows or out.shape[1] < heads * head_dim or q.shape[1] < heads * head_dim:
            raise KernelLibraryError("attention: q / out do not match rows x heads*head_dim")
        taken = torch.float32 if pieces > 1 else out.dtype
        if q.dtype != taken or kcache.dtype != out.dtype or vcache.dtype != out.dtype:
            raise KernelLibraryError("attention: q, out and the caches must share one dtype (pieces of q are float32)")
        if pieces > 1 and (cos_sin is None or piece_stride <= 0):
            raise KernelLibraryError("attention: pieces of q, k and v go with the folded rotation only")
        nb = kcache.shape[0]
        if tuple(kcache.shape) != (nb, kv_heads, block_size, head_dim) or \
                tuple(vcache.shape) != (nb, kv_heads, head_dim, block_size) or \
                not kcache.is_contiguous() or not vcache.is_contiguous():
            raise KernelLibraryError("attention: cache tensors do not have the paged layout")
        if seq_slot.dtype != torch.int32 or block_table.dtype != torch.int32 or block_table.dim() != 2:
            raise KernelLibraryError("attention: seq_slot and block_table must be int32 (table 2-D)")
        if decode and rows != batch:
            raise KernelLibraryError("attention: decode means one row per sequence")
        ws_n = 0
        if workspace is not None:
            if workspace.dtype != torch.float32 or not workspace.is_contiguous():
                raise KernelLibraryError("attention: workspace must be dense float32")
            ws_n = workspace.numel()
        ldk = ldv = 0
        if cos_sin is not None:
            self._dev(k_new, v_new, cos_sin)
            if k_new is None or v_new is None or not decode:
                raise KernelLibraryError("attention: the folded rotation needs the step's keys and values and a decoding step")
            if k_new.dtype != q.dtype or v_new.dtype != q.dtype or k_new.shape[0] != rows or v_new.shape[0] != rows \
                    or k_new.shape[1] < kv_heads * head_dim or v_new.shape[1] < kv_heads * head_dim:
                raise KernelLibraryError("attention: k_new / v_new do not match the rows or the kv width")
            if cos_sin.dtype != torch.float32 or tuple(cos_sin.shape) != (rows, head_dim // 2, 2) or not cos_sin.is_contiguous():
                raise KernelLibraryError("attention: cos_sin must be dense float32 [rows, head_dim/2, 2]")
            ldk, ldv = self._rows2d(k_new, "k_new"), self._rows2d(v_new, "v_new")
        tickets = self.tickets(q.device)
        folds = cos_sin is not None
        rc = self.lib.lq_attention(
            q.data_ptr(), self._rows2d(q, "q"), out.data_ptr(), self._rows2d(out, "out"), _code(out), rows, batch,
            heads, kv_heads, head_dim, row_pos.data_ptr(), row_seq.data_ptr(), seq_slot.data_ptr(), cu_rows.data_ptr(),
            block_table.data_ptr(), int(block_table.stride(0)), kcache.data_ptr(), vcache.data_ptr(), block_size,
            float(scale), window, 1 if decode else 0, max_len, 0 if workspace is None else workspace.data_ptr(), ws_n,
            tickets.data_ptr(), tickets.numel(), k_new.data_ptr() if folds else 0, v_new.data_ptr() if folds else 0,
            ldk, ldv, cos_sin.data_ptr() if folds else 0, 1 if uneven and decode else 0, pieces, piece_stride,
            1 if self.force_generic else 0, self.stream)
        if rc != 0:
            # a launch that did not run whole may have left tickets behind, and a later launch that found
            # them non-zero would never recognise its last workgroup: clear them (a fill kernel) before
            # the error goes up
            message = self.lib.lq_last_error().decode("utf-8", "replace")
            try:
                tickets.zero_()
            finally:
                raise KernelLibraryError(message)

    # ------------------------------------------------------------------ windowed attention with a sink
    def kv_store(self, k: torch.Tensor, v: torch.Tensor, kv_heads: int, key_dim: int, value_dim: int,
                 row_pos: torch.Tensor, row_seq: torch.Tensor, seq_slot: torch.Tensor, block_table: torch.Tensor,
                 kcache: torch.Tensor, vcache: torch.Tensor, block_size: int) -> None:
        """k [rows, kv_heads * key_dim] and v [rows, kv_heads * value_dim] go into the paged cache as they are, at
        the rows' positions (K [blocks, kv_heads, block_size, key_dim], V [blocks, kv_heads, value_dim, block_size])."""
        self._dev(k, v, row_pos, row_seq, seq_slot, block_table, kcache, vcache)
        rows = k.shape[0]
        self._i32(row_pos, "row_pos", rows)
        self._i32(row_seq, "row_seq", rows)
        self._check_paged(kcache, vcache, kv_heads, key_dim, value_dim, block_size, block_table, seq_slot, "kv_store")
        if v.shape[0] != rows or k.shape[1] != kv_heads * key_dim or v.shape[1] != kv_heads * value_dim \
                or k.dtype != kcache.dtype or v.dtype != kcache.dtype:
            raise KernelLibraryError("kv_store: k / v do not match the rows, the sizes or the cache's dtype")
        self._check(self.lib.lq_kv_store(
            _ptr(k), c_int(self._rows2d(k, "k")), _ptr(v), c_int(self._rows2d(v, "v")), c_int(_code(k)), c_int(rows),
            c_int(kv_heads), c_int(key_dim), c_int(value_dim), _ptr(row_pos), _ptr(row_seq), _ptr(seq_slot),
            _ptr(block_table), c_int(int(block_table.stride(0))), _ptr(kcache), _ptr(vcache), c_int(block_size),
            self.stream))

    @staticmethod
    def _check_paged(kcache, vcache, kv_heads, key_dim, value_dim, block_size, block_table, seq_slot, what) -> None:
        nb = kcache.shape[0]
        if tuple(kcache.shape) != (nb, kv_heads, block_size, key_dim) or \
                tuple(vcache.shape) != (nb, kv_heads, value_dim, block_size) or kcache.dtype != vcache.dtype or \
                not kcache.is_contiguous() or not vcache.is_contiguous():
            raise KernelLibraryError(f"{what}: cache tensors do not have the paged layout")
        if seq_slot.dtype != torch.int32 or block_table.dtype != torch.int32 or block_table.dim() != 2:
            raise KernelLibraryError(f"{what}: seq_slot and block_table must be int32 (table 2-D)")

    @query
    def sink_attention_workspace(self, dtype: torch.dtype, rows: int, batch: int, heads: int, kv_heads: int, key_dim: int,
                                 value_dim: int, block_size: int, window: int, keep_first: int, max_len: int) -> int:
        """Float32 entries of scratch with which `sink_attention` shares the keys of a launch of single tokens out
        over several workgroups a tile (0: it does not); `max_len`: an upper bound of the lengths."""
        if dtype not in _DTYPE_CODE:
            return 0
        self.lib.lq_sink_attention_workspace.restype = c_longlong
        return int(self.lib.lq_sink_attention_workspace(c_int(_DTYPE_CODE[dtype]), c_int(rows), c_int(batch), c_int(heads),
                                                        c_int(kv_heads), c_int(key_dim), c_int(value_dim),
                                                        c_int(block_size), c_int(window), c_int(keep_first),
                                                        c_int(max_len)))

    def sink_attention(self, q: torch.Tensor, out: torch.Tensor, heads: int, kv_heads: int, key_dim: int,
                       value_dim: int, row_pos: torch.Tensor, row_seq: torch.Tensor, seq_slot: torch.Tensor,
                       block_table: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, block_size: int,
                       scale: float, window: int = 0, keep_first: int = 0, sink: bool = True,
                       gate: Optional[torch.Tensor] = None, decode: bool = False, max_len: int = 0,
                       workspace: Optional[torch.Tensor] = None, sink_values: Optional[torch.Tensor] = None,
                       maps: int = 1) -> None:
        """Attention of the step's rows over their slots' cached keys: row at position p sees t <= p with
        p - t < window (0: all) or t < keep_first; with `sink` the softmax's denominator has one more term e^0;
        `gate` [rows, heads]: every head's result times the sigmoid of its entry.  Scores and probabilities
        are 32-bit.  out [rows, heads * value_dim] in the dtype of q and the cache.  `max_len` (an upper bound of the
        lengths) and `workspace` (`sink_attention_workspace(...)` floats) let a launch of single tokens share a tile's
        keys out over several workgroups (bfloat16 runs only).  `sink_values` (float32 [heads]): the sink's term is
        e^(its entry) for every query head, not e^0.  `maps` > 1: `kv_heads` counts key heads of which every `maps`
        neighbours share a value head; the cache is K [blocks, kv_heads / maps, block_size, maps * key_dim] (a row
        holds the neighbours' keys side by side) and V [blocks, kv_heads / maps, value_dim, block_size].  out may be
        float32 in a bfloat16 run."""
        self._dev(q, out, gate, row_pos, row_seq, seq_slot, block_table, kcache, vcache, sink_values)
        rows, batch = q.shape[0], seq_slot.numel()
        self._i32(row_pos, "row_pos", rows)
        self._i32(row_seq, "row_seq", rows)
        if maps < 1 or kv_heads % maps:
            raise KernelLibraryError(f"sink_attention: {kv_heads} key heads do not share value heads in runs of {maps}")
        self._check_paged(kcache, vcache, kv_heads // maps, key_dim * maps, value_dim, block_size, block_table, seq_slot,
                          "sink_attention")
        if q.shape[1] != heads * key_dim or tuple(out.shape) != (rows, heads * value_dim) \
                or out.dtype not in (q.dtype, torch.float32) or q.dtype != kcache.dtype:
            raise KernelLibraryError("sink_attention: q / out do not match the rows, the sizes or the cache's dtype")
        if sink_values is not None:
            if not sink:
                raise KernelLibraryError("sink_attention: learned sink scores without a sink")
            self._f32(sink_values, "sink_attention: sink_values", heads)
        if gate is not None and (tuple(gate.shape) != (rows, heads) or gate.dtype != q.dtype):
            raise KernelLibraryError("sink_attention: the gate is [rows, heads] in the dtype of q")
        if decode and rows != batch:
            raise KernelLibraryError("sink_attention: decode means one row per sequence")
        if workspace is not None:
            self._f32(workspace, "sink_attention: workspace", workspace.numel())
        self._check(self.lib.lq_sink_attention(
            _ptr(q), c_int(self._rows2d(q, "q")), _ptr(out), c_int(self._rows2d(out, "out")), _ptr(gate),
            c_int(0 if gate is None else self._rows2d(gate, "gate")), c_int(_code(q)), c_int(rows), c_int(batch),
            c_int(heads), c_int(kv_heads), c_int(key_dim), c_int(value_dim), _ptr(row_pos), _ptr(row_seq),
            _ptr(seq_slot), _ptr(block_table), c_int(int(block_table.stride(0))), _ptr(kcache), _ptr(vcache),
            c_int(block_size), c_float(scale), c_int(window), c_int(keep_first), c_int(1 if sink else 0),
            c_int(1 if self.force_generic else 0), c_int(max_len if workspace is not None else 0), _ptr(workspace),
            c_longlong(0 if workspace is None else workspace.numel()), _ptr(sink_values), c_int(maps),
            c_int(1 if out.dtype == torch.float32 else 0), self.stream))

    def diff_combine(self, both: torch.Tensor, out: torch.Tensor, heads: int, kv_heads: int, value_dim: int, lam: float,
                     eps: float, gain: float) -> None:
        """both float32 [rows, kv_heads, 2, heads / kv_heads, value_dim]: two attention results a query head over the
        same values.  out [rows, heads * value_dim] = (a1 - lam a2) / sqrt(mean((a1 - lam a2)^2) + eps) * gain, the
        mean over a head's value_dim."""
        rows, nb, ldb = self._mat(both, "diff_combine: both")
        ro, no, ldo = self._mat(out, "diff_combine: out")
        self._f32(both, "diff_combine: both")
        if heads % kv_heads or nb != 2 * heads * value_dim or (ro, no) != (rows, heads * value_dim):
            raise KernelLibraryError("diff_combine: both [rows, 2 heads value_dim] and out [rows, heads value_dim]")
        self._check(self.lib.lq_diff_combine(_ptr(both), c_int(ldb), _ptr(out), c_int(_code(out)), c_int(ldo), c_int(rows),
                                             c_int(heads), c_int(kv_heads), c_int(value_dim), c_float(lam), c_float(eps),
                                             c_float(gain), self.stream))

    # ------------------------------------------------------------------ recurrent mixers and what surrounds them
    _ACTIVATIONS = {"none": 0, "silu": 1, "relu": 2, "gelu_tanh": 3, "gelu": 4}

    @staticmethod
    def _f32(t: torch.Tensor, what: str, n: Optional[int] = None) -> None:
        if t.dtype != torch.float32 or not t.is_cuda or (n is not None and (t.numel() != n or not t.is_contiguous())):
            raise KernelLibraryError(f"{what}: a float32 tensor on the GPU" + (f" of {n} entries" if n is not None else ""))

    def dynamic_tanh(self, x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, alpha: torch.Tensor,
                     out: torch.Tensor, delta: Optional[torch.Tensor] = None, delta_scale: float = 1.0) -> None:
        """(x += delta_scale * delta;) out = tanh(alpha x) weight + bias; x float32, alpha a tensor of one entry."""
        rows, width, ldx = self._mat(x, "dynamic_tanh: x")
        self._f32(x, "dynamic_tanh: x")
        self._f32(weight, "dynamic_tanh: weight", width)
        self._f32(bias, "dynamic_tanh: bias", width)
        self._f32(alpha, "dynamic_tanh: alpha", 1)
        pieces, stride = self._pieces(delta, x, "dynamic_tanh")
        if delta is not None:
            self._f32(delta, "dynamic_tanh: delta")
        if not x.is_contiguous() or not out.is_contiguous() or tuple(out.shape) != (rows, width) or not out.is_cuda:
            raise KernelLibraryError("dynamic_tanh: x and out must be dense and of one shape")
        self._check(self.lib.lq_dynamic_tanh(_ptr(x), _ptr(delta), c_int(pieces), c_longlong(stride),
                                             c_float(delta_scale), _ptr(weight), _ptr(bias), _ptr(alpha), _ptr(out),
                                             c_int(_code(out)), c_int(rows), c_int(width), self.stream))

    def add_scaled(self, x: torch.Tensor, delta: torch.Tensor, scale: float) -> None:
        """x += scale * delta (delta shaped like x, or a stack of pieces whose sum is meant); float32."""
        self._f32(x, "add_scaled: x")
        self._f32(delta, "add_scaled: delta")
        pieces, stride = self._pieces(delta, x, "add_scaled")
        if not x.is_contiguous():
            raise KernelLibraryError("add_scaled: x must be dense")
        self._check(self.lib.lq_add_scaled(_ptr(x), _ptr(delta), c_int(pieces), c_longlong(stride), c_float(scale),
                                           c_longlong(x.numel()), self.stream))

    def activation(self, x: torch.Tensor, out: torch.Tensor, activation: str) -> None:
        """out = act(x), element by element in 32-bit; act: silu, relu, gelu_tanh or gelu (the exact one, with the error
        function)."""
        rows, inner, ld = self._mat(x, "activation: x")
        ro, wide, ldo = self._mat(out, "activation: out")
        if (ro, wide) != (rows, inner) or activation not in self._ACTIVATIONS or activation == "none":
            raise KernelLibraryError(f"activation: x {tuple(x.shape)}, out {tuple(out.shape)}, activation {activation!r}")
        self._check(self.lib.lq_glu(_ptr(x), c_int(_code(x)), c_int(ld), _ptr(out), c_int(_code(out)), c_int(ldo),
                                    c_int(rows), c_int(inner), c_int(self._ACTIVATIONS[activation]), _ptr(None), c_int(0),
                                    _ptr(None), c_int(0), c_int(0), self.stream))

    def glu(self, gate_up: torch.Tensor, out: torch.Tensor, activation: str, bias: Optional[torch.Tensor] = None,
            tail: int = 0, row_gate: Optional[torch.Tensor] = None) -> None:
        """out = act(gate) * up for gate_up [rows, 2 * inner] = [gate | up]; act: silu, relu or gelu_tanh.  `bias`
        (float32 [2 * inner]) is added to gate and up first.  With `tail` out is [rows, inner + tail] and its last
        columns become a one and then zeros (the next product's bias rides as one more column of its weight).
        `row_gate` (float32 [rows, 1], any row stride): a row's results times the sigmoid of its entry."""
        rows, two, ld = self._mat(gate_up, "glu: gate_up")
        ro, wide, ldo = self._mat(out, "glu: out")
        inner = wide - tail
        if ro != rows or tail < 0 or two != 2 * inner or activation not in self._ACTIVATIONS \
                or activation in ("none", "gelu"):
            raise KernelLibraryError(f"glu: gate_up {tuple(gate_up.shape)}, out {tuple(out.shape)}, activation {activation!r}")
        if bias is not None:
            self._f32(bias, "glu: bias", 2 * inner)
        ldrg = 0
        if row_gate is not None:
            rg, one, ldrg = self._mat(row_gate, "glu: row_gate")
            if (rg, one) != (rows, 1) or row_gate.dtype != torch.float32:
                raise KernelLibraryError("glu: the rows' gate is float32 [rows, 1]")
        self._check(self.lib.lq_glu(_ptr(gate_up), c_int(_code(gate_up)), c_int(ld), _ptr(out), c_int(_code(out)),
                                    c_int(ldo), c_int(rows), c_int(inner), c_int(self._ACTIVATIONS[activation]),
                                    _ptr(bias), c_int(tail), _ptr(row_gate), c_int(ldrg), c_int(1), self.stream))

    def causal_conv(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor,
                    out: torch.Tensor, row_pos: torch.Tensor, row_seq: torch.Tensor, seq_slot: torch.Tensor,
                    seq_start: torch.Tensor, seq_len: torch.Tensor, cu_rows: torch.Tensor, batch: int,
                    activation: str = "silu") -> None:
        """out[t, c] = act(bias[c] + sum_j weight[c, j] x[t - (taps - 1) + j, c]) along every sequence of the step;
        what lies before the step's rows comes from state [slots, taps - 1, channels] (a sequence's last inputs,
        zeros at its start), which is then moved on to the step's end.  All float32."""
        rows, ch, ldx = self._mat(x, "causal_conv: x")
        ro, co, ldo = self._mat(out, "causal_conv: out")
        taps = weight.shape[1] if weight.dim() == 2 else 0
        for t, what in ((x, "x"), (out, "out"), (state, "state")):
            self._f32(t, "causal_conv: " + what)
        self._f32(weight, "causal_conv: weight", ch * max(1, taps))
        if bias is not None:
            self._f32(bias, "causal_conv: bias", ch)
        if (ro, co) != (rows, ch) or taps < 1 or state.dim() != 3 or tuple(state.shape[1:]) != (max(1, taps - 1), ch) \
                or not state.is_contiguous() or activation not in self._ACTIVATIONS:
            raise KernelLibraryError("causal_conv: x, out [rows, channels], weight [channels, taps], "
                                     "state [slots, taps - 1, channels] do not fit")
        self._i32(row_pos, "row_pos", rows)
        self._i32(row_seq, "row_seq", rows)
        self._i32(seq_slot, "seq_slot", batch)
        self._i32(seq_start, "seq_start", batch)
        self._i32(cu_rows, "cu_rows", batch + 1)
        self._check(self.lib.lq_causal_conv(_ptr(x), c_int(ldx), _ptr(weight), _ptr(bias), _ptr(state), _ptr(out),
                                            c_int(ldo), c_int(rows), c_int(ch), c_int(taps), _ptr(row_seq), _ptr(row_pos),
                                            _ptr(seq_slot), _ptr(seq_start), _ptr(cu_rows), c_int(batch),
                                            c_int(self._ACTIVATIONS[activation]), self.stream))

    @query
    def ssd_scan_workspace(self, batch: int, heads: int, head_dim: int, n_state: int, max_rows: int) -> int:
        """Float32 entries of scratch with which `ssd_scan` runs this launch in segments (0: it does not)."""
        self.lib.lq_ssd_scan_workspace.restype = c_longlong
        return int(self.lib.lq_ssd_scan_workspace(c_int(batch), c_int(heads), c_int(head_dim), c_int(n_state),
                                                  c_int(max_rows)))

    def ssd_scan(self, x: torch.Tensor, b_in: torch.Tensor, c_in: torch.Tensor, dt: torch.Tensor, dt_bias: torch.Tensor,
                 a_log: torch.Tensor, d_skip: torch.Tensor, state: torch.Tensor, y: torch.Tensor, heads: int,
                 head_dim: int, n_state: int, groups: int, seq_slot: torch.Tensor, cu_rows: torch.Tensor,
                 batch: int, max_rows: int = 0, workspace: Optional[torch.Tensor] = None) -> None:
        """The Mamba-2 recurrence along every sequence of the step, token by token: with dt = softplus(dt + dt_bias),
        S <- exp(-exp(a_log) dt) S + dt B x^T and y = S^T C + d_skip x per head; state [slots, heads, head_dim,
        n_state] is read and left at the step's end.  All float32.  `max_rows` (the most rows a sequence brings)
        and `workspace` (`ssd_scan_workspace(...)` floats) let a launch of few long sequences run in segments."""
        rows = x.shape[0]
        for t, what, cols in ((x, "x", heads * head_dim), (b_in, "B", groups * n_state), (c_in, "C", groups * n_state),
                              (dt, "dt", heads), (y, "y", heads * head_dim)):
            self._f32(t, "ssd_scan: " + what)
            if self._mat(t, "ssd_scan: " + what)[:2] != (rows, cols):
                raise KernelLibraryError(f"ssd_scan: {what} must be [{rows}, {cols}], found {tuple(t.shape)}")
        for t, what in ((dt_bias, "dt_bias"), (a_log, "a_log"), (d_skip, "d_skip")):
            self._f32(t, "ssd_scan: " + what, heads)
        self._f32(state, "ssd_scan: state")
        if state.dim() != 4 or tuple(state.shape[1:]) != (heads, head_dim, n_state) or not state.is_contiguous():
            raise KernelLibraryError("ssd_scan: state must be dense [slots, heads, head_dim, n_state]")
        self._i32(seq_slot, "seq_slot", batch)
        self._i32(cu_rows, "cu_rows", batch + 1)
        if workspace is not None:
            self._f32(workspace, "ssd_scan: workspace", workspace.numel())
        ld = self._rows2d
        self._check(self.lib.lq_ssd_scan(_ptr(x), c_int(ld(x, "x")), _ptr(b_in), c_int(ld(b_in, "B")), _ptr(c_in),
                                         c_int(ld(c_in, "C")), _ptr(dt), c_int(ld(dt, "dt")), _ptr(dt_bias), _ptr(a_log),
                                         _ptr(d_skip), _ptr(state), _ptr(y), c_int(ld(y, "y")), c_int(heads),
                                         c_int(head_dim), c_int(n_state), c_int(groups), _ptr(seq_slot), _ptr(cu_rows),
                                         c_int(batch), c_int(max_rows if workspace is not None else 0), _ptr(workspace),
                                         c_longlong(0 if workspace is None else workspace.numel()), self.stream))

    def delta_scan(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, beta: torch.Tensor, a: torch.Tensor,
                   dt_bias: torch.Tensor, a_log: torch.Tensor, state: torch.Tensor, out: torch.Tensor, heads: int,
                   kv_heads: int, key_dim: int, value_dim: int, q_scale: float, unit_eps: float,
                   seq_slot: torch.Tensor, cu_rows: torch.Tensor, batch: int, channel_decay: bool = False) -> None:
        """The gated delta rule along every sequence of the step, token by token: q and k made unit vectors per
        head (x / sqrt(sum x^2 + unit_eps)), q times q_scale, beta = sigmoid(beta), g = exp(-exp(a_log)
        softplus(a + dt_bias)); S <- g S, u = beta (v - S^T k), S <- S + k u^T, out = S^T q.  state [slots, heads,
        value_dim, key_dim].  All float32.  q and k are overwritten with their unit vectors.  The decay is one number
        a head (a [rows, heads], dt_bias [heads]) or, with `channel_decay`, one for every key channel of every head
        (a [rows, heads * key_dim], dt_bias [heads * key_dim]), multiplying the state's rows of that channel."""
        rows = q.shape[0]
        n_decay = heads * key_dim if channel_decay else heads
        for t, what, cols in ((q, "q", kv_heads * key_dim), (k, "k", kv_heads * key_dim), (v, "v", heads * value_dim),
                              (beta, "beta", heads), (a, "a", n_decay), (out, "out", heads * value_dim)):
            self._f32(t, "delta_scan: " + what)
            if self._mat(t, "delta_scan: " + what)[:2] != (rows, cols):
                raise KernelLibraryError(f"delta_scan: {what} must be [{rows}, {cols}], found {tuple(t.shape)}")
        self._f32(dt_bias, "delta_scan: dt_bias", n_decay)
        self._f32(a_log, "delta_scan: a_log", heads)
        self._f32(state, "delta_scan: state")
        if state.dim() != 4 or tuple(state.shape[1:]) != (heads, value_dim, key_dim) or not state.is_contiguous():
            raise KernelLibraryError("delta_scan: state must be dense [slots, heads, value_dim, key_dim]")
        self._i32(seq_slot, "seq_slot", batch)
        self._i32(cu_rows, "cu_rows", batch + 1)
        ld = self._rows2d
        self._check(self.lib.lq_delta_scan(_ptr(q), c_int(ld(q, "q")), _ptr(k), c_int(ld(k, "k")), _ptr(v),
                                           c_int(ld(v, "v")), _ptr(beta), c_int(ld(beta, "beta")), _ptr(a),
                                           c_int(ld(a, "a")), _ptr(dt_bias), _ptr(a_log), _ptr(state), _ptr(out),
                                           c_int(ld(out, "out")), c_int(heads), c_int(kv_heads), c_int(key_dim),
                                           c_int(value_dim), c_float(q_scale), c_float(unit_eps), _ptr(seq_slot),
                                           _ptr(cu_rows), c_int(batch), c_int(rows), c_int(1 if channel_decay else 0),
                                           self.stream))

    def gated_rmsnorm(self, y: torch.Tensor, z: torch.Tensor, weight: torch.Tensor, eps: float, group: int,
                      out: torch.Tensor, gate_first: bool = True, gate: str = "silu") -> None:
        """RMS norm of y [rows, n] in parts of `group` columns, each by its own root mean square, with a gate
        silu(z): gate_first: (y silu(z)) normed, times weight; else y normed, times weight, times silu(z).  The
        weight has n entries, or fewer that repeat (one weight for every part).  `gate` "sigmoid": sigmoid(z) in the
        place of silu(z)."""
        if gate not in ("silu", "sigmoid"):
            raise KernelLibraryError(f"gated_rmsnorm: the gate is 'silu' or 'sigmoid', found {gate!r}")
        rows, n, ldy = self._mat(y, "gated_rmsnorm: y")
        rz, nz, ldz = self._mat(z, "gated_rmsnorm: z")
        ro, no, ldo = self._mat(out, "gated_rmsnorm: out")
        self._f32(y, "gated_rmsnorm: y")
        self._f32(z, "gated_rmsnorm: z")
        self._f32(weight, "gated_rmsnorm: weight", weight.numel())
        if (rz, nz) != (rows, n) or (ro, no) != (rows, n) or group <= 0 or n % group:
            raise KernelLibraryError("gated_rmsnorm: y, z and out must be [rows, n] with n a multiple of the group")
        self._check(self.lib.lq_gated_rmsnorm(_ptr(y), c_int(ldy), _ptr(z), c_int(ldz), _ptr(weight),
                                              c_int(weight.numel()), c_float(eps), c_int(group), _ptr(out),
                                              c_int(_code(out)), c_int(ldo), c_int(rows), c_int(n),
                                              c_int(1 if gate_first else 0), c_int(1 if gate == "sigmoid" else 0),
                                              self.stream))

    def rmsnorm_mean(self, stack: torch.Tensor, weights, eps: float, out: torch.Tensor) -> None:
        """out = mean over i of stack[i] / rms(stack[i]) * weights[i], row by row; stack [n, rows, width] float32."""
        self._f32(stack, "rmsnorm_mean: stack")
        self._f32(out, "rmsnorm_mean: out")
        if stack.dim() != 3 or not stack.is_contiguous() or not out.is_contiguous() \
                or tuple(out.shape) != tuple(stack.shape[1:]) or len(weights) != stack.shape[0] or not 1 <= len(weights) <= 4:
            raise KernelLibraryError("rmsnorm_mean: a dense stack [n, rows, width] of 1 to 4 branches, a weight for each")
        n, rows, width = stack.shape
        for w in weights:
            self._f32(w, "rmsnorm_mean: weight", width)
        ws = [_ptr(w) for w in weights] + [c_void_p(0)] * (4 - n)
        self._check(self.lib.lq_rmsnorm_mean(_ptr(stack), c_int(n), *ws, c_float(eps), _ptr(out), c_int(rows),
                                             c_int(width), self.stream))

    # ------------------------------------------------------------------ bigram embedding, norm on a sublayer's result,
    # ------------------------------------------------------------------ gated linear attention, latent attention, experts
    def bigram_add(self, x: torch.Tensor, table: torch.Tensor, tokens: torch.Tensor, last: torch.Tensor, buckets: int,
                   mul_prev: int, mul_cur: int, vocab: int, row_pos: torch.Tensor, row_seq: torch.Tensor,
                   seq_slot: torch.Tensor, cu_rows: torch.Tensor, batch: int) -> None:
        """x[r] += table[(previous * mul_prev + token * mul_cur) mod buckets] (row `buckets` for a sequence's first
        token); the token before a step's first row comes from last[slot], which then takes the step's last token."""
        self._dev(x, table, tokens, last, row_pos, row_seq, seq_slot, cu_rows)
        rows, width = x.shape
        if x.dtype != torch.float32 or not x.is_contiguous() or table.dim() != 2 or not table.is_contiguous() \
                or tuple(table.shape) != (buckets + 1, width):
            raise KernelLibraryError(f"bigram_add: x dense float32 [rows, width], the table dense [{buckets + 1}, width]")
        if last.dtype != torch.int32 or not last.is_contiguous() or last.numel() != last.shape[0]:
            raise KernelLibraryError("bigram_add: the last tokens are a dense int32 entry a slot")
        for t, what, n in ((tokens, "tokens", rows), (row_pos, "row_pos", rows), (row_seq, "row_seq", rows),
                           (seq_slot, "seq_slot", batch), (cu_rows, "cu_rows", batch + 1)):
            self._i32(t, what, n)
        self._check(self.lib.lq_bigram_add(_ptr(x), _ptr(table), c_int(_code(table)), _ptr(tokens), _ptr(last),
                                           c_longlong(buckets), c_longlong(mul_prev), c_longlong(mul_cur), c_int(vocab),
                                           c_int(rows), c_int(width), _ptr(row_pos), _ptr(row_seq), _ptr(seq_slot),
                                           _ptr(cu_rows), self.stream))

    def rmsnorm_residual(self, x: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float,
                         rounded: Optional[torch.Tensor] = None) -> None:
        """x += y / sqrt(mean(y^2) + eps) * weight, row by row (x and y float32); `rounded`, where given, takes the
        new x in its own dtype."""
        self._dev(x, y, weight, rounded)
        rows, width = x.shape
        if x.dtype != torch.float32 or y.dtype != torch.float32 or tuple(y.shape) != (rows, width) \
                or not x.is_contiguous() or not y.is_contiguous():
            raise KernelLibraryError("rmsnorm_residual: x and y must be dense float32 of one shape")
        self._f32(weight, "rmsnorm_residual: weight", width)
        if rounded is not None and (tuple(rounded.shape) != (rows, width) or not rounded.is_contiguous()):
            raise KernelLibraryError("rmsnorm_residual: rounded must be dense and shaped like x")
        self._check(self.lib.lq_rmsnorm_residual(_ptr(x), _ptr(y), _ptr(weight), c_float(eps), _ptr(rounded),
                                                 c_int(_code(rounded) if rounded is not None else 0), c_int(rows),
                                                 c_int(width), self.stream))

    def rmsnorm_cols(self, src: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor) -> None:
        """out = src / sqrt(mean(src^2) + eps) * weight, row by row; src float32 [rows, n] and out [rows, n] may
        each be a run of columns of a wider row."""
        rows, n, lds = self._mat(src, "rmsnorm_cols: src")
        ro, no, ldo = self._mat(out, "rmsnorm_cols: out")
        if src.dtype != torch.float32 or (ro, no) != (rows, n):
            raise KernelLibraryError("rmsnorm_cols: src float32 [rows, n], out [rows, n]")
        self._f32(weight, "rmsnorm_cols: weight", n)
        self._check(self.lib.lq_rmsnorm_cols(_ptr(src), c_int(lds), _ptr(weight), c_float(eps), _ptr(out),
                                             c_int(_code(out)), c_int(ldo), c_int(rows), c_int(n), self.stream))

    def rotary(self, src: torch.Tensor, out: torch.Tensor, heads: int, size: int, out_head_stride: int, dims: int,
               interleaved: bool, freqs: torch.Tensor, magnitude: float, row_pos: torch.Tensor) -> None:
        """Head h of row r: src[r, h size .. + size) (float32) goes to out[r, h out_head_stride .. + size), its first
        `dims` entries rotated by row_pos[r] * freqs (float64 [dims / 2]) in half-split pairs (j, j + dims / 2) or
        interleaved pairs (2 j, 2 j + 1), cos and sin times `magnitude`.  `out` starts at the first entry written
        and may be a run of columns of a wider row."""
        rows, ns, lds = self._mat(src, "rotary: src")
        ro, no, ldo = self._mat(out, "rotary: out")
        self._i32(row_pos, "row_pos", rows)
        if src.dtype != torch.float32 or ns != heads * size or ro != rows or no < (heads - 1) * out_head_stride + size:
            raise KernelLibraryError("rotary: src float32 [rows, heads * size], out with room for every head's vector")
        if freqs.dtype != torch.float64 or not freqs.is_cuda or not freqs.is_contiguous() or freqs.numel() != dims // 2:
            raise KernelLibraryError(f"rotary: {dims // 2} float64 frequencies on the GPU")
        self._check(self.lib.lq_rotary(_ptr(src), c_int(lds), _ptr(out), c_int(_code(out)), c_int(ldo), c_int(rows),
                                       c_int(heads), c_int(size), c_int(out_head_stride), c_int(dims),
                                       c_int(1 if interleaved else 0), _ptr(freqs), c_float(magnitude), _ptr(row_pos),
                                       self.stream))

    def rotary_qkv(self, src: torch.Tensor, q_out: torch.Tensor, k_out: torch.Tensor, v_out: torch.Tensor, heads: int,
                   kv_heads: int, key_dim: int, value_dim: int, dims: int, interleaved: bool,
                   freqs: Optional[torch.Tensor], magnitude: float, norm_eps: Optional[float],
                   row_pos: torch.Tensor, value_width: int = 0) -> None:
        """src float32 [rows, (heads + kv_heads) key_dim + kv_heads value_dim] = [queries | keys | values] goes to
        q_out, k_out and v_out in their dtype: of every query and key head the first `dims` entries rotated by
        row_pos[r] * freqs (float64 [dims / 2]; pairing and magnitude as `rotary`), then, with `norm_eps` not None,
        the head divided by its root mean square over key_dim (eps inside the root); values pass.  `value_width` > 0:
        the values are so many entries a row, not kv_heads * value_dim (key heads that share a value head)."""
        rows, ns, lds = self._mat(src, "rotary_qkv: src")
        rq, nq, ldq = self._mat(q_out, "rotary_qkv: q")
        rk, nk, ldk = self._mat(k_out, "rotary_qkv: k")
        rv, nv, ldv = self._mat(v_out, "rotary_qkv: v")
        self._i32(row_pos, "row_pos", rows)
        vw = value_width if value_width > 0 else kv_heads * value_dim
        if src.dtype != torch.float32 or ns != (heads + kv_heads) * key_dim + vw \
                or (rq, nq) != (rows, heads * key_dim) or (rk, nk) != (rows, kv_heads * key_dim) \
                or (rv, nv) != (rows, vw) or not q_out.dtype == k_out.dtype == v_out.dtype:
            raise KernelLibraryError("rotary_qkv: src float32 [rows, q | k | v], outputs of one dtype with their sizes")
        if dims and (freqs is None or freqs.dtype != torch.float64 or not freqs.is_cuda or not freqs.is_contiguous()
                     or freqs.numel() != dims // 2):
            raise KernelLibraryError(f"rotary_qkv: {dims // 2} float64 frequencies on the GPU")
        self._check(self.lib.lq_rotary_qkv(_ptr(src), c_int(lds), _ptr(q_out), c_int(ldq), _ptr(k_out), c_int(ldk),
                                           _ptr(v_out), c_int(ldv), c_int(_code(q_out)), c_int(rows), c_int(heads),
                                           c_int(kv_heads), c_int(key_dim), c_int(value_dim), c_int(dims),
                                           c_int(1 if interleaved else 0), _ptr(freqs if dims else None),
                                           c_float(magnitude), c_float(-1.0 if norm_eps is None else norm_eps),
                                           _ptr(row_pos), c_int(value_width), self.stream))

    def postnorm_residual(self, x: torch.Tensor, y: torch.Tensor, scales, weight: torch.Tensor, eps: float,
                          extra: Optional[torch.Tensor] = None, next_weight: Optional[torch.Tensor] = None,
                          next_eps: float = 0.0, h: Optional[torch.Tensor] = None) -> None:
        """With y the sum of scales[i] * y[i] over a stack [n, rows, width] of 1 to 4 pieces (or y [rows, width] and
        one scale): x += y / sqrt(mean(y^2) + eps) * weight; then x += extra, where given; then, where `h` is given,
        h = x / sqrt(mean(x^2) + next_eps) * next_weight in the dtype of h.  x, y, extra float32."""
        rows, width = x.shape
        self._f32(x, "postnorm_residual: x", rows * width)
        self._f32(y, "postnorm_residual: y")
        pieces, stride = self._pieces(y, x, "postnorm_residual")
        if len(scales) != pieces or not 1 <= pieces <= 4:
            raise KernelLibraryError(f"postnorm_residual: {pieces} pieces and {len(scales)} scales (1 to 4 of each)")
        self._f32(weight, "postnorm_residual: weight", width)
        if extra is not None:
            self._f32(extra, "postnorm_residual: extra", rows * width)
        if (h is None) != (next_weight is None):
            raise KernelLibraryError("postnorm_residual: the next norm's weight and its output come together")
        if h is not None:
            self._f32(next_weight, "postnorm_residual: next weight", width)
            self._dev(h)
            if tuple(h.shape) != (rows, width) or not h.is_contiguous():
                raise KernelLibraryError("postnorm_residual: h must be dense and shaped like x")
        sc = [float(v) for v in scales] + [0.0] * (4 - pieces)
        self._check(self.lib.lq_postnorm_residual(_ptr(x), _ptr(y), c_int(pieces), c_longlong(stride), c_float(sc[0]),
                                                  c_float(sc[1]), c_float(sc[2]), c_float(sc[3]), _ptr(weight),
                                                  c_float(eps), _ptr(extra), _ptr(next_weight), c_float(next_eps),
                                                  _ptr(h), c_int(_code(h) if h is not None else 0), c_int(rows),
                                                  c_int(width), self.stream))

    def scale(self, x: torch.Tensor, factor: float) -> None:
        """x *= factor (dense float32)."""
        self._f32(x, "scale: x", x.numel())
        self._check(self.lib.lq_scale(_ptr(x), c_float(factor), c_longlong(x.numel()), self.stream))

    def linear_heads(self, x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, heads: int, out_head_stride: int) -> None:
        """A product a head: out[r, h out_head_stride .. + N) = x[r, h K .. + K) . w[h]^T with w [heads, N, K]: one
        launch for bfloat16 operands with K in 16s, else a product a head."""
        rows, kx, ldx = self._mat(x, "linear_heads: x")
        ro, no, ldc = self._mat(out, "linear_heads: out")
        if w.dim() != 3 or not w.is_contiguous() or not w.is_cuda or w.shape[0] != heads or kx != heads * w.shape[2] \
                or ro != rows or no < (heads - 1) * out_head_stride + w.shape[1] or out_head_stride < w.shape[1] \
                or x.dtype != w.dtype:
            raise KernelLibraryError(f"linear_heads: x {tuple(x.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} do not fit")
        n, k = int(w.shape[1]), int(w.shape[2])
        if not self.force_generic and self.lib.lq_linear_heads_accepts(_ptr(x), _ptr(w), c_int(_code(x)), c_int(k), c_int(ldx)):
            self._check(self.lib.lq_linear_heads(_ptr(x), c_int(ldx), _ptr(w), _ptr(out), c_int(_code(x)), c_int(_code(out)),
                                                 c_int(ldc), c_int(rows), c_int(heads), c_int(n), c_int(k),
                                                 c_int(out_head_stride), self.stream))
            return
        xe, we, oe = x.element_size(), w.element_size(), out.element_size()
        cx, co = _code(x), _code(out)
        generic = 1 if self.force_generic else 0
        for h in range(heads):
            rc = self.lib.lq_linear(x.data_ptr() + h * k * xe, w.data_ptr() + h * n * k * we,
                                    out.data_ptr() + h * out_head_stride * oe, cx, co, rows, n, k, ldx, k, ldc, 1, 0,
                                    generic, 0, self.stream)
            if rc:
                self._check(rc)

    @query
    def gla_scan_workspace(self, batch: int, heads: int, key_dim: int, value_dim: int, max_rows: int) -> int:
        """Float32 entries of scratch with which `gla_scan` runs this launch in segments (0: it does not)."""
        self.lib.lq_gla_scan_workspace.restype = c_longlong
        return int(self.lib.lq_gla_scan_workspace(c_int(batch), c_int(heads), c_int(value_dim), c_int(key_dim),
                                                  c_int(max_rows)))

    def gla_scan(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, z: torch.Tensor, bias: torch.Tensor,
                 state: torch.Tensor, out: torch.Tensor, heads: int, key_dim: int, value_dim: int, q_scale: float,
                 inv_tau: float, seq_slot: torch.Tensor, cu_rows: torch.Tensor, batch: int, max_rows: int = 0,
                 workspace: Optional[torch.Tensor] = None) -> None:
        """Gated linear attention along every sequence of the step, token by token: with the decay a =
        sigmoid(z + bias)^inv_tau for every key channel, S <- diag(a) S + k v^T and out = S^T (q q_scale) per head;
        state [slots, heads, value_dim, key_dim] is read and left at the step's end.  All float32.  `max_rows` (the
        most rows a sequence brings) and `workspace` (`gla_scan_workspace(...)` floats) let a launch of few long
        sequences run in segments side by side (every segment from zero, the end states chained with the products
        of the segments' decays, the segments again from their true starts)."""
        rows = q.shape[0]
        for t, what, cols in ((q, "q", heads * key_dim), (k, "k", heads * key_dim), (z, "z", heads * key_dim),
                              (v, "v", heads * value_dim), (out, "out", heads * value_dim)):
            self._f32(t, "gla_scan: " + what)
            if self._mat(t, "gla_scan: " + what)[:2] != (rows, cols):
                raise KernelLibraryError(f"gla_scan: {what} must be [{rows}, {cols}], found {tuple(t.shape)}")
        self._f32(bias, "gla_scan: bias", heads * key_dim)
        self._f32(state, "gla_scan: state")
        if state.dim() != 4 or tuple(state.shape[1:]) != (heads, value_dim, key_dim) or not state.is_contiguous():
            raise KernelLibraryError("gla_scan: state must be dense [slots, heads, value_dim, key_dim]")
        self._i32(seq_slot, "seq_slot", batch)
        self._i32(cu_rows, "cu_rows", batch + 1)
        if workspace is not None:
            self._f32(workspace, "gla_scan: workspace", workspace.numel())
        ld = self._rows2d
        self._check(self.lib.lq_gla_scan(_ptr(q), c_int(ld(q, "q")), _ptr(k), c_int(ld(k, "k")), _ptr(v),
                                         c_int(ld(v, "v")), _ptr(z), c_int(ld(z, "z")), _ptr(bias), _ptr(state), _ptr(out),
                                         c_int(ld(out, "out")), c_int(heads), c_int(key_dim), c_int(value_dim),
                                         c_float(q_scale), c_float(inv_tau), _ptr(seq_slot), _ptr(cu_rows), c_int(batch),
                                         c_int(max_rows if workspace is not None else 0), _ptr(workspace),
                                         c_longlong(0 if workspace is None else workspace.numel()), self.stream))

    def moe_route(self, logits: torch.Tensor, route: torch.Tensor, top: int, renormalize: bool = False,
                  correction: Optional[torch.Tensor] = None, groups: int = 0, keep: int = 0, scoring: str = "sigmoid",
                  group_mark: str = "top2", renormalize_eps: float = 0.0,
                  identity: Optional[torch.Tensor] = None) -> None:
        """route[r, e] = sigmoid(logits[r, e]) for the `top` experts with the largest scores (the lower index on a
        tie; divided by the chosen scores' sum with `renormalize`), -1 for the others.  float32.  With `correction`
        (float32 [experts]) the choice goes by score + correction, the weights stay the scores.  With `groups` > 1
        the experts form that many equal groups of neighbours and only experts of the `keep` groups whose two largest
        choice scores sum highest can be chosen (`group_mark` "max": whose largest choice score is highest).
        `scoring` "softmax": the scores are softmax(logits) over all columns.  `renormalize_eps` is added to the chosen
        scores' sum before the division.  `identity` (float32 [rows, n]): the last n columns of the logits are experts
        without tensors; their weights (-1: not chosen) go there and `route` is [rows, experts - n]."""
        rows, experts, ldz = self._mat(logits, "moe_route: logits")
        self._f32(logits, "moe_route: logits")
        n_ident = 0
        if identity is not None:
            n_ident = identity.shape[-1]
            self._f32(identity, "moe_route: identity", rows * n_ident)
        if scoring not in ("sigmoid", "softmax") or group_mark not in ("top2", "max"):
            raise KernelLibraryError(f"moe_route: scoring {scoring!r}, group_mark {group_mark!r}")
        self._f32(route, "moe_route: route", rows * (experts - n_ident))
        if correction is not None:
            self._f32(correction, "moe_route: correction", experts)
        self._check(self.lib.lq_moe_route(_ptr(logits), c_int(ldz), _ptr(route), c_int(rows), c_int(experts), c_int(top),
                                          c_int(1 if renormalize else 0), _ptr(correction), c_int(groups), c_int(keep),
                                          c_int(1 if scoring == "softmax" else 0), c_int(1 if group_mark == "max" else 0),
                                          c_float(renormalize_eps), _ptr(identity), c_int(n_ident), self.stream))

    def moe_identity(self, h: torch.Tensor, weights: torch.Tensor, out: torch.Tensor) -> None:
        """out [rows, width] (float32) += h * (the sum of the row's entries of `weights` [rows, n] that are not
        negative): the share of experts that hand their input on."""
        rows, width, ldh = self._mat(h, "moe_identity: h")
        ro, wo, ldo = self._mat(out, "moe_identity: out")
        self._f32(out, "moe_identity: out")
        if (ro, wo) != (rows, width) or weights.dim() != 2 or weights.shape[0] != rows:
            raise KernelLibraryError("moe_identity: h and out [rows, width], weights [rows, n]")
        self._f32(weights, "moe_identity: weights", rows * weights.shape[1])
        self._check(self.lib.lq_moe_identity(_ptr(h), c_int(_code(h)), c_int(ldh), _ptr(weights), c_int(weights.shape[1]),
                                             _ptr(out), c_int(ldo), c_int(rows), c_int(width), self.stream))

    def moe_glu(self, gu: torch.Tensor, route: torch.Tensor, out: torch.Tensor, experts: int, ff: int, limit: float,
                weight_input: bool = True, activation: str = "clamped_swish") -> None:
        """gu [rows, experts * 2 ff] float32 (every expert's gate then up), route [rows, experts]; out [rows,
        experts * ff]: for a chosen expert with weight w, g = min(w gate, limit), u = clamp(w up, -limit, limit),
        y = g sigmoid(1.702 g) (u + 1) (with `weight_input` false w multiplies y instead); 0 for the others.
        `activation` "silu": y = silu(gate) up, no clamps."""
        if activation not in ("clamped_swish", "silu"):
            raise KernelLibraryError(f"moe_glu: unknown activation {activation!r}")
        rows, ng, ldg = self._mat(gu, "moe_glu: gu")
        ro, no, ldo = self._mat(out, "moe_glu: out")
        self._f32(gu, "moe_glu: gu")
        self._f32(route, "moe_glu: route", rows * experts)
        if ng != experts * 2 * ff or (ro, no) != (rows, experts * ff):
            raise KernelLibraryError("moe_glu: gu [rows, experts * 2 ff] and out [rows, experts * ff]")
        self._check(self.lib.lq_moe_glu(_ptr(gu), c_longlong(ldg), _ptr(route), _ptr(out), c_int(_code(out)),
                                        c_longlong(ldo), c_int(rows), c_int(experts), c_int(ff), c_float(limit),
                                        c_int(1 if weight_input else 0), c_int(1 if activation == "silu" else 0),
                                        self.stream))

    def weight_rows(self, w, start: int, n: int):
        """Rows start .. start + n of a product weight as a weight of its own: a view of a dense one; of a packed
        one the same run of its memory, where the rows are whole groups of eight and a matrix of that size is
        packed at all (else None: the caller keeps the weight dense)."""
        if not getattr(w, "packed", False):
            return w[start : start + n]
        rows, k = w.shape
        if start % 8 or n % 8 or start + n > rows or \
                not self.lib.lq_weight_packable(c_int(_DTYPE_CODE[w.dtype]), c_int(n), c_int(k)):
            return None
        return PackedWeight(w.data.view(-1)[start * k : (start + n) * k].view(n, k), n, k)

    def moe_sort(self, route: torch.Tensor, counts: torch.Tensor, order: torch.Tensor, weight: torch.Tensor,
                 place_of: torch.Tensor) -> None:
        """The chosen (row, expert) couples of route [rows, experts] (a weight, or -1), expert by expert with rows
        ascending: counts[e] rows of expert e, order[place] = row, weight[place] = its weight, place_of[row, e] =
        place or -1."""
        rows, experts = route.shape
        self._f32(route, "moe_sort: route", rows * experts)
        self._f32(weight, "moe_sort: weight")
        self._i32(counts, "counts", experts)
        self._i32(place_of, "place_of", rows * experts)
        if order.dtype != torch.int32 or not order.is_contiguous() or not weight.is_contiguous() \
                or order.numel() != weight.numel() or order.numel() < rows:
            raise KernelLibraryError("moe_sort: order (int32) and weight (float32) hold a place for every chosen couple")
        self._dev(route, counts, order, weight, place_of)
        self._check(self.lib.lq_moe_sort(_ptr(route), c_int(rows), c_int(experts), _ptr(counts), _ptr(order), _ptr(weight),
                                         _ptr(place_of), self.stream))

    def moe_gather(self, src: torch.Tensor, order: torch.Tensor, dst: torch.Tensor, n: int) -> None:
        """dst[i] = src[order[i]] for the first n places."""
        rows, width, ld = self._mat(src, "moe_gather: src")
        if dst.dtype != src.dtype or dst.dim() != 2 or dst.shape[1] != width or not dst.is_contiguous() or dst.shape[0] < n \
                or order.numel() < n or order.dtype != torch.int32 or not dst.is_cuda:
            raise KernelLibraryError("moe_gather: dst dense [>= n, width] in the dtype of src, order int32")
        self._check(self.lib.lq_moe_gather(_ptr(src), c_int(_code(src)), c_int(ld), _ptr(order), _ptr(dst), c_int(n),
                                           c_int(width), self.stream))

    def moe_scatter(self, ys: torch.Tensor, place_of: torch.Tensor, out: torch.Tensor) -> None:
        """out[r] = the sum over the experts e that row r chose, in ascending order, of ys[place_of[r, e]]."""
        rows, width, ldo = self._mat(out, "moe_scatter: out")
        self._f32(ys, "moe_scatter: ys")
        self._f32(out, "moe_scatter: out")
        if place_of.dtype != torch.int32 or place_of.dim() != 2 or place_of.shape[0] != rows or not place_of.is_contiguous() \
                or ys.dim() != 2 or ys.shape[1] != width or not ys.is_contiguous():
            raise KernelLibraryError("moe_scatter: ys dense [places, width], place_of int32 [rows, experts]")
        self._check(self.lib.lq_moe_scatter(_ptr(ys), _ptr(place_of), c_int(place_of.shape[1]), _ptr(out), c_int(ldo),
                                            c_int(rows), c_int(width), self.stream))

    # ------------------------------------------------------------------ sampling
    @property
    def penalty_window(self) -> int:
        """Width of the ring of recent ids that the sampling kernels take (the library's constant)."""
        return int(self.lib.lq_penalty_window())

    def apply_penalty(self, logits: torch.Tensor, seq_slot: torch.Tensor, recent: torch.Tensor,
                      recent_n: torch.Tensor, penalty: float) -> None:
        """Repetition penalty on the distinct ids in each sequence's ring of recent tokens, in place."""
        self._dev(logits, seq_slot, recent, recent_n)
        rows, vocab = logits.shape
        self._i32(seq_slot, "seq_slot", rows)
        if logits.dtype != torch.float32 or recent.dtype != torch.int32 or recent_n.dtype != torch.int32 \
                or recent.dim() != 2 or recent.shape[1] != self.penalty_window or not recent.is_contiguous():
            raise KernelLibraryError(f"penalty: logits float32, ring int32 [slots, {self.penalty_window}], counters int32")
        self._check(self.lib.lq_apply_penalty(_ptr(logits), c_int(self._rows2d(logits, "logits")), c_int(rows),
                                              c_int(vocab), _ptr(seq_slot), _ptr(recent), _ptr(recent_n),
                                              c_float(penalty), self.stream))

    def argmax(self, logits: torch.Tensor, out: torch.Tensor, scratch: torch.Tensor,
               seq_slot: Optional[torch.Tensor] = None, recent: Optional[torch.Tensor] = None,
               recent_n: Optional[torch.Tensor] = None) -> None:
        """out[r] = first maximal index of logits[r]; the token is pushed into the ring if one is given.
        `scratch`: int64 with at least 32 entries a row."""
        self._dev(logits, out, scratch, seq_slot, recent, recent_n)
        rows, vocab = logits.shape
        self._i32(out, "argmax out", rows)
        if logits.dtype != torch.float32:
            raise KernelLibraryError("argmax: logits must be float32")
        if scratch.dtype != torch.int64 or not scratch.is_contiguous() or scratch.numel() < 32 * rows:
            raise KernelLibraryError(f"argmax: scratch must be dense int64 with at least {32 * rows} entries")
        if recent is not None:
            self._i32(seq_slot, "seq_slot", rows)
        self._check(self.lib.lq_argmax(_ptr(logits), c_int(self._rows2d(logits, "logits")), c_int(rows),
                                       c_int(vocab), _ptr(seq_slot), _ptr(out), _ptr(recent), _ptr(recent_n),
                                       _ptr(scratch), self.stream))

    def sample(self, logits: torch.Tensor, out: torch.Tensor, seq_slot: torch.Tensor, temperature: float,
               top_k: int, top_p: float, rng_key: torch.Tensor, rng_ctr: torch.Tensor,
               recent: Optional[torch.Tensor] = None, recent_n: Optional[torch.Tensor] = None,
               kept_count: Optional[torch.Tensor] = None, kept_mass: Optional[torch.Tensor] = None,
               scratch: Optional[torch.Tensor] = None) -> None:
        """Temperature sampling with top-k and top-p; each sequence's counter moves on by one.  With
        `scratch` (uint8, `sample_scratch_bytes(rows)`) and a small top-k the row is worked on in parts
        by many compute units instead of one."""
        self._dev(logits, out, seq_slot, rng_key, rng_ctr, recent, recent_n, kept_count, kept_mass, scratch)
        if scratch is not None and (scratch.dtype != torch.uint8 or not scratch.is_contiguous()):
            raise KernelLibraryError("sample: scratch must be dense uint8")
        rows, vocab = logits.shape
        self._i32(out, "sample out", rows)
        self._i32(seq_slot, "seq_slot", rows)
        if logits.dtype != torch.float32 or rng_key.dtype != torch.int64 or rng_ctr.dtype != torch.int64:
            raise KernelLibraryError("sample: logits float32, generator key and counter int64")
        if kept_count is not None:
            self._i32(kept_count, "kept_count", rows)
        if kept_mass is not None and (kept_mass.dtype != torch.float64 or kept_mass.numel() < rows):
            raise KernelLibraryError("sample: kept_mass must be float64 with one entry a row")
        self._check(self.lib.lq_sample(_ptr(logits), c_int(self._rows2d(logits, "logits")), c_int(rows),
                                       c_int(vocab), _ptr(seq_slot), c_float(temperature), c_int(top_k),
                                       c_float(top_p), _ptr(rng_key), _ptr(rng_ctr), _ptr(recent), _ptr(recent_n),
                                       _ptr(out), _ptr(kept_count), _ptr(kept_mass), _ptr(scratch),
                                       c_longlong(scratch.numel() if scratch is not None else 0), self.stream))

    @query
    def sample_scratch_bytes(self, rows: int) -> int:
        self.lib.lq_sample_scratch_bytes.restype = c_longlong
        return int(self.lib.lq_sample_scratch_bytes(c_int(rows)))

    def advance(self, row_pos: torch.Tensor, seq_start: torch.Tensor, seq_len: torch.Tensor, batch: int) -> None:
        """Positions and lengths of a decoding batch move on by one."""
        self._dev(row_pos, seq_start, seq_len)
        for t in (row_pos, seq_start, seq_len):
            self._i32(t, "advance", batch)
        self._check(self.lib.lq_advance(_ptr(row_pos), _ptr(seq_start), _ptr(seq_len), c_int(batch), self.stream))

    # ------------------------------------------------------------------ HIP graphs
    def graph_begin(self) -> None:
        self._check(self.lib.lq_graph_begin(self.stream))

    def graph_end(self) -> int:
        handle = c_void_p(0)
        self._check(self.lib.lq_graph_end(self.stream, ctypes.byref(handle)))
        return int(handle.value)

    def graph_launch(self, handle: int) -> None:
        self._check(self.lib.lq_graph_launch(c_void_p(handle), self.stream))

    def graph_destroy(self, handle: int) -> None:
        self._check(self.lib.lq_graph_destroy(c_void_p(handle)))
