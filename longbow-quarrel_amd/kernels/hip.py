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
ABI_VERSION = 5  # lq_abi_version() of the library these wrappers were written for
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

    def embed(self, table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor) -> None:
        """out[r, :] = float32(table[tokens[r], :]); zeros where tokens[r] is no row of the table"""
        self._dev(table, tokens, out)
        rows, width = out.shape
        self._i32(tokens, "embed tokens", rows)
        if out.dtype != torch.float32 or not out.is_contiguous() or not table.is_contiguous():
            raise KernelLibraryError("embed: out must be dense float32, the table dense")
        if table.dim() != 2 or table.shape[1] != width:
            raise KernelLibraryError(f"embed: table {tuple(table.shape)} does not match width {width}")
        self._check(self.lib.lq_embed(_ptr(table), c_int(_code(table)), _ptr(tokens), _ptr(out),
                                      c_int(rows), c_int(width), c_int(table.shape[0]), c_int(_packed(table)),
                                      self.stream))

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
