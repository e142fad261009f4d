"""`HipTensor`: the host-side mirror of the reference's GPU tensor backends for the GEMM +
broadcast/map hot path, on top of the C ABI of libam_hip.so.

It occupies the slot of `CudaTensor` (src/arraymancer/tensor/data_structure.nim:29-67): a shape /
strides / offset view over reference-counted device storage, with the same operator set
(src/arraymancer/tensor/operators_blas_l2l3_cuda.nim, operators_blas_l1_cuda.nim,
operators_broadcasted_cuda.nim, shapeshifting_cuda.nim, init_cuda.nim), extended to the four
element types of the CPU path (float32, float64, int32, int64) and to arbitrary strides.

Reference operator          here
  t.cuda / t.cpu            toHip(ndarray) / t.toCpu()
  a * b (matrices)          a * b          (also a @ b);   gemm(alpha, A, B, beta, C)
  a + b, a - b, +=, -=      same
  t * s, s * t, t / s       same (scalar s)
  a +. b  a -. b  a *. b  a /. b  a mod b      bc_add / bc_sub / bc_mul / bc_div / bc_mod  (OPERATORS["+."] ...)
  a +.= b ... (rhs broadcast only)              a.bc_iadd(b) / bc_isub / bc_imul / bc_idiv
  map2_inline(a, b, <expr>)                     map2(op_name, a, b) for the enumerated bodies
  t.transpose, t[slices], t.broadcast(shape)    same, metadata only
Python has no `+.` token, hence the names; the argument order and error behaviour follow the
reference (ValueError for shape mismatches, IndexError for matrix dimension mismatches).
"""
from __future__ import annotations

import ctypes
from typing import Sequence

import numpy as np

from . import _lib
from . import metadata as md
from ._lib import CMP, CTYPE, EPI, OP, OP3, PRED, RED, SFX, UOP, check, i64_array
from .metadata import Layout, Step


class HipStorage:
    """Owns one device allocation; freed when the last view goes away
    (the reference frees in the ref-tracker's destructor, data_structure.nim:60-67)."""

    __slots__ = ("ptr", "nelems", "itemsize", "__weakref__")

    def __init__(self, nelems: int, itemsize: int):
        L = _lib.load()
        out = ctypes.c_void_p()
        check(L.am_hip_malloc(ctypes.c_size_t(nelems * itemsize), ctypes.byref(out)))
        self.ptr = out.value or 0
        self.nelems = nelems
        self.itemsize = itemsize

    def __del__(self):
        ptr, self.ptr = getattr(self, "ptr", 0), 0
        if ptr:
            try:
                rc = _lib.load().am_hip_free(ctypes.c_void_p(ptr))
            except Exception:  # interpreter shutdown
                return
            if rc != 0:        # a destructor cannot raise: say so instead of leaking silently
                import warnings
                warnings.warn(f"am_hip_free failed ({rc}): {_lib.last_error()}", ResourceWarning)


# Unsigned element types ride the kernels of their signed twins, like the reference's GEMM overload for
# uint32 | uint64 | uint | int (laser/primitives/matrix_multiplication/gemm.nim:275-307: the pointers are cast onto the
# int32 / int64 kernels). In the rings Z/2^32 and Z/2^64 the bits of + - * (hence of GEMM, gemv, dot, sums and
# products, x*y+z) do not depend on how the operands are read; division, remainder, comparisons, min / max and
# everything float-valued do, and are refused for these types.
_UNSIGNED_TWIN = {np.dtype(np.uint32): "i32", np.dtype(np.uint64): "i64"}
_RING_OPS = frozenset(("add", "sub", "mul"))
_RING_UOPS = frozenset(("copy", "neg"))
_RING_OP3 = frozenset(("muladd", "addmul"))
_RING_RED = frozenset(("sum", "product"))


def _dtype_sfx(dtype) -> str:
    try:
        return SFX[np.dtype(dtype)]
    except KeyError:
        if np.dtype(dtype) in _UNSIGNED_TWIN:
            return _UNSIGNED_TWIN[np.dtype(dtype)]
        raise TypeError(f"HipTensor supports float32, float64, int32, int64 (and uint32 / uint64 for + - * and "
                        f"products), not {dtype}")


def _ring_scalar(sfx: str, dtype, value):
    """The scalar argument of a ring operation as the kernel's C type: an unsigned value above the signed twin's
    range is passed as the same bits (ctypes integer types wrap instead of raising)."""
    return CTYPE[sfx](int(value) if np.dtype(dtype).kind in "iu" else value)


# Element types a HipTensor can hold as the RESULT of a map whose body changes the type (Tensor[bool] of the
# comparisons, one byte per element; classify's FloatClass ordinals): views and toCpu work, arithmetic does not.
_RESULT_ONLY = (np.dtype(np.bool_), np.dtype(np.uint8))


class HipTensor:
    __slots__ = ("layout", "storage", "dtype", "pool_geometry")

    def __init__(self, layout: Layout, storage: HipStorage, dtype):
        self.layout = layout
        self.storage = storage
        self.dtype = np.dtype(dtype)

    # ------------------------------------------------------------------ metadata
    @property
    def shape(self):
        return self.layout.shape

    @property
    def strides(self):
        return self.layout.strides

    @property
    def offset(self):
        return self.layout.offset

    @property
    def rank(self):
        return self.layout.rank

    @property
    def size(self):
        return self.layout.size

    @property
    def sfx(self) -> str:
        try:
            return SFX[self.dtype]
        except KeyError:
            if self.dtype in _UNSIGNED_TWIN:
                raise TypeError(f"this operation reads the sign of its operands and is not defined on a HipTensor of "
                                f"{self.dtype}: unsigned tensors support + - *, matrix products, sums and products")
            raise TypeError(f"no arithmetic is defined on a HipTensor of {self.dtype}")

    @property
    def ring_sfx(self) -> str:
        """Kernel suffix for an operation of the ring Z/2^n (+ - * and what is built from them): an unsigned tensor
        takes the kernels of its signed twin (gemm.nim:275-307)."""
        return _UNSIGNED_TWIN.get(self.dtype) or self.sfx

    def data_ptr(self) -> int:
        """Device address of element [0, 0, ...] (get_offset_ptr, data_structure.nim:206-211)."""
        return self.storage.ptr + self.layout.offset * self.dtype.itemsize

    def is_C_contiguous(self):
        return md.is_C_contiguous(self.layout)

    def is_F_contiguous(self):
        return md.is_F_contiguous(self.layout)

    def isContiguous(self):
        return self.is_C_contiguous() or self.is_F_contiguous()

    def __repr__(self):
        return f"HipTensor[{self.dtype}](shape={list(self.shape)}, strides={list(self.strides)}, offset={self.offset})"

    def pretty(self, precision: int = -1, specifier: str = "") -> str:
        """The reference's `pretty` / `$` for a device tensor (src/arraymancer/tensor/display_cuda.nim:19-36):
        a host copy laid out by the CPU printer (display.nim:19-115), under a header that names this
        type and backend. `specifier`: "" (table), "||", "[]", "[:]", "<>", "<:>" and their header forms."""
        from . import display
        return display.pretty_array(np.ascontiguousarray(self.toCpu()), "HipTensor", "Hip", precision, specifier)

    def __str__(self):
        return self.pretty()

    # ------------------------------------------------------------------ views (no data movement)
    def transpose(self) -> "HipTensor":
        return HipTensor(md.transpose(self.layout), self.storage, self.dtype)

    @property
    def T(self):
        return self.transpose()

    def squeeze(self, axis: int | None = None) -> "HipTensor":
        """Without the dimensions of extent 1, or without the one at `axis` (shapeshifting.nim:396-413)."""
        return HipTensor(md.squeeze(self.layout, axis), self.storage, self.dtype)

    def unsqueeze(self, axis: int) -> "HipTensor":
        """With a dimension of extent 1 inserted at `axis` (shapeshifting.nim:415-424)."""
        return HipTensor(md.unsqueeze(self.layout, axis), self.storage, self.dtype)

    def permute(self, *dims) -> "HipTensor":
        """The dimensions in a new order, same data (src/arraymancer/tensor/shapeshifting.nim:207-226)."""
        if len(dims) == 1 and not isinstance(dims[0], int):
            dims = tuple(dims[0])
        return HipTensor(md.permute(self.layout, dims), self.storage, self.dtype)

    def __getitem__(self, key) -> "HipTensor":
        return HipTensor(md.py_index(self.layout, key), self.storage, self.dtype)

    def slice_(self, *steps: Step) -> "HipTensor":
        """Slicing in the reference's notation: Step(first, last, step) with inclusive ends."""
        return HipTensor(md.slicer(self.layout, steps), self.storage, self.dtype)

    def broadcast(self, shape: Sequence[int]) -> "HipTensor":
        return HipTensor(md.broadcast(self.layout, shape), self.storage, self.dtype)

    bc = broadcast

    def reshape(self, *shape) -> "HipTensor":
        if len(shape) == 1 and not isinstance(shape[0], int):
            shape = tuple(shape[0])
        n = 1
        for s in shape:
            n *= s
        if n != self.size:
            raise ValueError(f"The total number of elements in the old ({self.size}) and the new ({n}) "
                             f"reshaped tensor must be the same")
        src = self if self.is_C_contiguous() else self.clone()
        lay = md.contiguous(shape)
        return HipTensor(Layout(lay.shape, lay.strides, src.layout.offset), src.storage, self.dtype)

    # ------------------------------------------------------------------ transfers and copies
    def toCpu(self) -> np.ndarray:
        """Blocking copy back. Like the reference's `cpu` (init_cuda.nim:43-59) the whole storage
        is copied and shape / strides / offset are kept, so the result is the same view of the
        same bytes (a NumPy strided view here)."""
        host = np.empty(self.storage.nelems, dtype=self.dtype)
        if self.storage.nelems:
            check(_lib.load().am_hip_memcpy_d2h(host.ctypes.data, ctypes.c_void_p(self.storage.ptr),
                                                ctypes.c_size_t(host.nbytes)))
        if self.size == 0:
            return np.empty(self.shape, dtype=self.dtype)
        it = self.dtype.itemsize
        lo, hi = md.extent_in_storage(self.layout)
        assert 0 <= lo and hi < self.storage.nelems
        return np.lib.stride_tricks.as_strided(host[self.layout.offset:], shape=self.shape,
                                               strides=tuple(s * it for s in self.strides))

    def clone(self) -> "HipTensor":
        """Fresh C-contiguous copy (device-side strided gather)."""
        out = empty(self.shape, self.dtype)
        _unary_into("copy", out, self)
        return out

    def asContiguous(self) -> "HipTensor":
        return self if self.is_C_contiguous() else self.clone()

    # ------------------------------------------------------------------ operators
    def __mul__(self, other):
        if isinstance(other, HipTensor):
            return matmul(self, other)
        return scalar_op("mul", self, other)

    def __rmul__(self, other):
        return scalar_op("mul", self, other, scalar_on_left=True)

    __matmul__ = lambda self, other: matmul(self, other)

    def __truediv__(self, other):
        if isinstance(other, HipTensor):
            raise TypeError("tensor / tensor is spelled bc_div (`/.`)")
        return scalar_op("div", self, other)

    def __add__(self, other):
        _check_elementwise(self, other)
        return map2("add", self, other)

    def __sub__(self, other):
        _check_elementwise(self, other)
        return map2("sub", self, other)

    def __iadd__(self, other):
        _check_elementwise(self, other)
        _binary_into("add", self, self, other)
        return self

    def __isub__(self, other):
        _check_elementwise(self, other)
        _binary_into("sub", self, self, other)
        return self

    def __imul__(self, scalar):
        _scalar_into("mul", self, self, scalar, False)
        return self

    def __itruediv__(self, scalar):
        _scalar_into("div", self, self, scalar, False)
        return self

    def __neg__(self):
        return unary("neg", self)

    # in-place broadcast forms: only the right-hand side may be broadcast
    # (src/arraymancer/tensor/operators_broadcasted.nim:65-102)
    def bc_iadd(self, other):
        return _bc_inplace("add", self, other)

    def bc_isub(self, other):
        return _bc_inplace("sub", self, other)

    def bc_imul(self, other):
        return _bc_inplace("mul", self, other)

    def bc_idiv(self, other):
        return _bc_inplace("div", self, other)

    def bc_ipow(self, exponent):
        """`^.=`: in-place pow(x, exponent), float tensors, scalar exponent
        (src/arraymancer/tensor/operators_broadcasted.nim:178-182)."""
        _float_scalar("^.=", self, exponent)
        if self.size:
            _scalar_into("pow", self, self, exponent, False)
        return self


# ---------------------------------------------------------------------- construction
def empty(shape: Sequence[int], dtype) -> HipTensor:
    """newTensorUninit on the device: row-major, uninitialised."""
    dtype = np.dtype(dtype)
    if dtype not in _RESULT_ONLY:
        _dtype_sfx(dtype)
    lay = md.contiguous(shape)
    return HipTensor(lay, HipStorage(lay.size, dtype.itemsize), dtype)


def zeros(shape: Sequence[int], dtype) -> HipTensor:
    t = empty(shape, dtype)
    if t.size:
        check(_lib.load().am_hip_memset(ctypes.c_void_p(t.storage.ptr), 0,
                                        ctypes.c_size_t(t.size * t.dtype.itemsize)))
    return t


def toHip(arr) -> HipTensor:
    """Host -> device. Row-major on the device, like CPU tensors (the CUDA backend's forced
    column-major copy, init_cuda.nim:31, is not kept). A non-contiguous ndarray is packed on
    the host first; strided device views are made with transpose / slicing on the HipTensor."""
    arr = np.asarray(arr)
    _dtype_sfx(arr.dtype)
    host = np.ascontiguousarray(arr)
    t = empty(host.shape, host.dtype)
    if host.size:
        check(_lib.load().am_hip_memcpy_h2d(ctypes.c_void_p(t.storage.ptr), host.ctypes.data,
                                            ctypes.c_size_t(host.nbytes)))
    return t


def broadcast(val, shape: Sequence[int], dtype=None) -> HipTensor:
    """`broadcast(val, shape)` (src/arraymancer/tensor/shapeshifting.nim:136-176): a tensor of `shape` whose every
    element is `val` - ONE element of storage, every stride 0. Like the reference's, it must not be written through
    (all positions share the element); `clone` / `asContiguous` materialise it. A HipTensor as first argument is the
    tensor form (explicit broadcast of its size-1 dimensions)."""
    if isinstance(val, HipTensor):
        return val.broadcast(shape)
    if dtype is None:
        dtype = np.asarray(val).dtype
        if dtype == np.dtype(np.int_) and dtype not in SFX:
            dtype = np.dtype(np.int64)
    dtype = np.dtype(dtype)
    _dtype_sfx(dtype)
    one = toHip(np.full((1,), val, dtype=dtype))
    shape = tuple(int(d) for d in shape)
    if any(d < 0 for d in shape) or len(shape) > _lib.AM_MAXRANK:
        raise ValueError(f"broadcast: invalid shape {list(shape)}")
    return HipTensor(Layout(shape, (0,) * len(shape), 0), one.storage, dtype)


def sync() -> None:
    check(_lib.load().am_hip_sync())


class Graph:
    """Records the device operations issued inside `with Graph() as g:` into a HIP graph instead
    of running them; `g.launch()` replays the sequence with one call. Allocation during the block is
    served from the allocator's cache of freed blocks only (`Graph.record(fn)` prepares it with a
    rehearsal); results that are read after a replay must live in tensors made before the block, e.g. with
    `empty` and the `gemm(alpha, A, B, beta, C)` / `apply2` / `_into` forms. A tensor that goes out of scope inside the
    block is kept alive by the graph (the library holds its block until the graph is destroyed); tensors
    recorded in the graph and dropped after the block must outlive the replays - pass them to `keep()`
    to tie their lifetime to the graph's."""

    def __init__(self):
        self._exec = ctypes.c_void_p()

    def __enter__(self):
        check(_lib.load().am_hip_graph_begin())
        return self

    def __exit__(self, exc_type, exc, tb):
        rc = _lib.load().am_hip_graph_end(ctypes.byref(self._exec))
        if exc_type is None:
            check(rc)
        return False

    def launch(self):
        check(_lib.load().am_hip_graph_launch(self._exec))

    @staticmethod
    def record(fn) -> "Graph":
        """A graph of everything `fn()` issues, temporaries included. `fn` runs twice: once as a rehearsal with the
        allocator holding back every block that is freed (afterwards its cache has one block per allocation `fn`
        makes, and the library workspace its final size), then under capture, where allocation is served from that
        cache. `fn` must only issue device work (no read-backs, uploads or `zeros`) on tensors that outlive the graph."""
        L = _lib.load()
        check(L.am_hip_alloc_hold(1))
        try:
            fn()
        finally:
            check(L.am_hip_alloc_hold(0))
        with Graph() as g:
            fn()
        return g

    def keep(self, *tensors):
        """Holds a reference to the storage of each tensor for as long as this graph exists."""
        self._kept = getattr(self, "_kept", []) + [t.storage for t in tensors]
        return self

    def __del__(self):
        ex, self._exec = getattr(self, "_exec", None), None
        if ex:
            try:
                _lib.load().am_hip_graph_destroy(ex)
            except Exception:
                pass


# ---------------------------------------------------------------------- checks
def _same_dtype(*ts):
    d = ts[0].dtype
    for t in ts[1:]:
        if t.dtype != d:
            raise TypeError(f"element types differ: {d} and {t.dtype}")
    return d


def _check_elementwise(a: HipTensor, b: HipTensor):
    """check_elementwise (src/arraymancer/tensor/private/p_checks.nim:59-62)."""
    if not isinstance(b, HipTensor):
        raise TypeError("operand must be a HipTensor")
    if a.shape != b.shape:
        raise ValueError(f"Both Tensors should have the same shape. Left-hand side has shape "
                         f"{list(a.shape)} while right-hand side has shape {list(b.shape)}")


# ---------------------------------------------------------------------- GEMM
class DigitPlanes:
    """The base-256 digit planes of an integer matrix, split once on the device for products that reuse the matrix (a
    weight matrix): `digits_prepare(W, side)` makes them, `gemm(..., a_digits=..., b_digits=...)` uses them in place
    of splitting that operand in every call. A snapshot: prepare again after the matrix changes. Released with the
    object (or `release()`)."""

    def __init__(self, handle: int, side: int, shape, dtype):
        self.handle, self.side, self.shape, self.dtype = handle, side, tuple(shape), np.dtype(dtype)

    def release(self):
        h, self.handle = getattr(self, "handle", 0), 0
        if h:
            check(_lib.load().am_hip_digits_release(ctypes.c_void_p(h)))

    def __del__(self):
        try:
            self.release()
        except Exception:
            pass


def digits_prepare(t: HipTensor, side: str | int = "right") -> DigitPlanes:
    """Splits the int32 / int64 (or unsigned twin) matrix `t` into its digit planes for later products in which it is
    the "left" ([M x K]) or "right" ([K x N]) operand. Any strides; blocking."""
    if t.rank != 2:
        raise ValueError("digits_prepare: the operand must be a matrix")
    sfx = t.ring_sfx
    if sfx not in ("i32", "i64"):
        raise TypeError("digits_prepare is defined for integer tensors")
    s = {"left": 0, "right": 1}.get(side, side)
    out = ctypes.c_void_p()
    check(getattr(_lib.load(), f"am_hip_digits_prepare_{sfx}")(
        int(s), t.shape[0], t.shape[1], ctypes.c_void_p(t.data_ptr()), t.strides[0], t.strides[1], ctypes.byref(out)))
    return DigitPlanes(out.value, int(s), t.shape, t.dtype)


def gemm(alpha, A: HipTensor, B: HipTensor, beta, C: HipTensor, epilogue="none", bias: HipTensor | None = None,
         a_digits: DigitPlanes | None = None, b_digits: DigitPlanes | None = None):
    """C <- alpha * A * B + beta * C in place (C may be any non-overlapping strided view).
    src/arraymancer/tensor/operators_blas_l2l3.nim:58-81. Optional fused epilogue
    ("bias", "relu", "bias_relu") with `bias` broadcastable to C's shape (float types). a_digits / b_digits: the digit
    planes of an integer A / B split ahead of time (`digits_prepare`)."""
    dtype = _same_dtype(A, B, C)
    if A.rank != 2 or B.rank != 2 or C.rank != 2:
        raise ValueError("gemm: A, B and C must be matrices")
    M, K = A.shape
    K2, N = B.shape
    if K != K2:   # check_matmat raises IndexDefect, src/arraymancer/tensor/private/p_checks.nim:159-167
        raise IndexError(f"Number of columns in the first matrix: {K}, must be the same as the number "
                         f"of rows in the second matrix: {K2}")
    if C.shape != (M, N):
        raise IndexError(f"gemm: C has shape {list(C.shape)}, expected {[M, N]}")
    L = _lib.load()
    sfx = C.ring_sfx
    args = [M, N, K, _ring_scalar(sfx, dtype, alpha), ctypes.c_void_p(A.data_ptr()), A.strides[0], A.strides[1],
            ctypes.c_void_p(B.data_ptr()), B.strides[0], B.strides[1], _ring_scalar(sfx, dtype, beta),
            ctypes.c_void_p(C.data_ptr()), C.strides[0], C.strides[1]]
    epi = EPI[epilogue] if isinstance(epilogue, str) else int(epilogue)
    if a_digits is not None or b_digits is not None:
        if sfx not in ("i32", "i64") or epi != 0:
            raise TypeError("prepared digit planes belong to integer products without an epilogue")
        for d, side in ((a_digits, 0), (b_digits, 1)):
            if d is not None and (d.side != side or d.dtype != dtype):
                raise ValueError("gemm: digit planes prepared for the other side of a product, or for another element type")
        ha = ctypes.c_void_p(a_digits.handle) if a_digits is not None else None
        hb = ctypes.c_void_p(b_digits.handle) if b_digits is not None else None
        check(getattr(L, f"am_hip_gemm_prepared_{sfx}")(*args[:7], ha, *args[7:10], hb, *args[10:]))
        return C
    if epi != 0:
        if sfx not in ("f32", "f64"):
            raise TypeError("fused epilogues are defined for float tensors")
        bptr, brs, bcs = None, 0, 0
        if epi & 1:
            if bias is None:
                raise ValueError("bias epilogue needs a bias tensor")
            _same_dtype(C, bias)
            bb = bias.broadcast((M, N))
            bptr, brs, bcs = ctypes.c_void_p(bb.data_ptr()), bb.strides[0], bb.strides[1]
        check(getattr(L, f"am_hip_gemm_ex_{sfx}")(*args, epi, bptr, brs, bcs))
    else:
        check(getattr(L, f"am_hip_gemm_{sfx}")(*args))
    return C


def matmul(a: HipTensor, b: HipTensor) -> HipTensor:
    """`*` (src/arraymancer/tensor/operators_blas_l2l3.nim:88-100): matrix-matrix, or
    matrix-vector (run as an N = 1 product); anything else is a ValueError."""
    _same_dtype(a, b)
    if a.rank == 2 and b.rank == 2:
        if a.shape[1] != b.shape[0]:
            raise IndexError(f"Number of columns in the first matrix: {a.shape[1]}, must be the same as the "
                             f"number of rows in the second matrix: {b.shape[0]}")
        out = empty((a.shape[0], b.shape[1]), a.dtype)
        return gemm(1, a, b, 0, out)
    if a.rank == 2 and b.rank == 1:
        if a.shape[1] != b.shape[0]:
            raise IndexError(f"Number of columns in the matrix: {a.shape[1]}, must be the same as the "
                             f"number of rows in the vector: {b.shape[0]}")
        out = empty((a.shape[0],), a.dtype)
        return gemv(1, a, b, 0, out)
    raise ValueError("Matrix-Matrix or Matrix-Vector multiplication valid only if first Tensor is a "
                     "Matrix and second is a Matrix or Vector")


def gemv(alpha, A: HipTensor, x: HipTensor, beta, y: HipTensor) -> HipTensor:
    """y <- alpha * A * x + beta * y (src/arraymancer/tensor/operators_blas_l2l3.nim:24-56)."""
    _same_dtype(A, x, y)
    if A.rank != 2 or x.rank != 1 or y.rank != 1:
        raise ValueError("gemv: A must be a matrix, x and y vectors")
    if A.shape[1] != x.shape[0]:   # check_matvec, p_checks.nim:169-178
        raise IndexError(f"Number of columns in the matrix: {A.shape[1]}, must be the same as the number "
                         f"of rows in the vector: {x.shape[0]}")
    if y.shape[0] != A.shape[0]:
        raise IndexError(f"gemv: y has {y.shape[0]} elements, expected {A.shape[0]}")
    sfx = y.ring_sfx
    check(getattr(_lib.load(), f"am_hip_gemv_{sfx}")(
        A.shape[0], A.shape[1], _ring_scalar(sfx, y.dtype, alpha), ctypes.c_void_p(A.data_ptr()), A.strides[0], A.strides[1],
        ctypes.c_void_p(x.data_ptr()), x.strides[0], _ring_scalar(sfx, y.dtype, beta), ctypes.c_void_p(y.data_ptr()), y.strides[0]))
    return y


def dot(a: HipTensor, b: HipTensor):
    """Vector-vector scalar product, returned to the host
    (src/arraymancer/tensor/operators_blas_l1.nim:27-38)."""
    _same_dtype(a, b)
    if a.rank != 1 or b.rank != 1 or a.shape != b.shape:
        raise ValueError(f"dot: both operands must be vectors of the same length, got {list(a.shape)} and {list(b.shape)}")
    sfx = a.ring_sfx
    out = CTYPE[sfx]()
    check(getattr(_lib.load(), f"am_hip_dot_{sfx}")(
        a.shape[0], ctypes.c_void_p(a.data_ptr()), a.strides[0], ctypes.c_void_p(b.data_ptr()), b.strides[0],
        ctypes.byref(out)))
    return _host_scalar(a.dtype, out.value)


def _host_scalar(dtype, value):
    """A kernel's scalar result as the tensor's element type (an unsigned tensor's result arrives in its signed twin)."""
    dtype = np.dtype(dtype)
    if dtype in _UNSIGNED_TWIN:
        return dtype.type(int(value) % (1 << (8 * dtype.itemsize)))
    return dtype.type(value)


def gemm_batched(alpha, A: HipTensor, B: HipTensor, beta, C: HipTensor, epilogue="none", bias: HipTensor | None = None):
    """C[z] <- alpha * A[z] * B[z] + beta * C[z] for rank-3 operands [batch, rows, cols] in one
    launch. A or B of rank 2 is shared by the whole batch (batch stride 0)."""
    dtype = _same_dtype(A, B, C)
    if C.rank != 3 or A.rank not in (2, 3) or B.rank not in (2, 3):
        raise ValueError("gemm_batched: C must be [batch, M, N]; A and B [batch, ., .] or shared matrices")
    batch, M, N = C.shape
    a_sh, a_st, a_b = (A.shape[-2:], A.strides[-2:], A.strides[0] if A.rank == 3 else 0)
    b_sh, b_st, b_b = (B.shape[-2:], B.strides[-2:], B.strides[0] if B.rank == 3 else 0)
    if (A.rank == 3 and A.shape[0] != batch) or (B.rank == 3 and B.shape[0] != batch):
        raise IndexError("gemm_batched: batch sizes differ")
    K = a_sh[1]
    if a_sh[0] != M or b_sh != (K, N):
        raise IndexError(f"gemm_batched: shapes {list(A.shape)} x {list(B.shape)} -> {list(C.shape)} do not agree")
    sfx, ct = C.sfx, CTYPE[C.sfx]
    epi = EPI[epilogue] if isinstance(epilogue, str) else int(epilogue)
    bptr, brs, bcs = None, 0, 0
    if epi & 1:
        if bias is None:
            raise ValueError("bias epilogue needs a bias tensor")
        bb = bias.broadcast((M, N))
        bptr, brs, bcs = ctypes.c_void_p(bb.data_ptr()), bb.strides[0], bb.strides[1]
    check(getattr(_lib.load(), f"am_hip_gemm_batched_{sfx}")(
        batch, M, N, K, ct(alpha), ctypes.c_void_p(A.data_ptr()), a_st[0], a_st[1], a_b,
        ctypes.c_void_p(B.data_ptr()), b_st[0], b_st[1], b_b, ct(beta),
        ctypes.c_void_p(C.data_ptr()), C.strides[1], C.strides[2], C.strides[0], epi, bptr, brs, bcs))
    return C


def im2col(x: HipTensor, kernel_size, padding=(0, 0), stride=(1, 1)) -> HipTensor:
    """[N, C, H, W] -> [N, C*kH*kW, H_out*W_out] on the device, whole batch in one launch
    (src/arraymancer/nn_primitives/fallback/conv.nim:18-54 does one image per call on the host)."""
    if x.rank != 4:
        raise ValueError("im2col: input must be [N, C, H, W]")
    N, C, H, W = x.shape
    (kh, kw), (ph, pw), (sh, sw) = kernel_size, padding, stride
    ho, wo = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
    col = empty((N, C * kh * kw, ho * wo), x.dtype)
    check(getattr(_lib.load(), f"am_hip_im2col_{x.sfx}")(
        N, C, H, W, kh, kw, ph, pw, sh, sw, ctypes.c_void_p(x.data_ptr()), *x.strides, ctypes.c_void_p(col.data_ptr())))
    return col


def im2col_folded(x: HipTensor, kernel_size, padding=(0, 0), stride=(1, 1)) -> HipTensor:
    """[N, C, H, W] -> [C*kH*kW, N * H_out*W_out]: the column matrices of all images side by side (image n's columns
    from n * H_out*W_out on), so that a product over the whole batch is one GEMM. Same entries as `im2col`."""
    if x.rank != 4:
        raise ValueError("im2col: input must be [N, C, H, W]")
    N, C, H, W = x.shape
    (kh, kw), (ph, pw), (sh, sw) = kernel_size, padding, stride
    ho, wo = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
    col = empty((C * kh * kw, N * ho * wo), x.dtype)
    check(getattr(_lib.load(), f"am_hip_im2col_strided_{x.sfx}")(
        N, C, H, W, kh, kw, ph, pw, sh, sw, ctypes.c_void_p(x.data_ptr()), *x.strides, ctypes.c_void_p(col.data_ptr()),
        ho * wo, N * ho * wo))
    return col


def col2im(col: HipTensor, channels: int, height: int, width: int, kernel_size, padding=(0, 0), stride=(1, 1)) -> HipTensor:
    """col2im (src/arraymancer/nn_primitives/fallback/conv.nim:55-79): [C*kH*kW, H_out*W_out] -> [C, H, W], or for a
    batch [N, C*kH*kW, H_out*W_out] -> [N, C, H, W] in one launch; pixels covered by several columns are summed."""
    (kh, kw), (ph, pw), (sh, sw) = kernel_size, padding, stride
    ho, wo = (height + 2 * ph - kh) // sh + 1, (width + 2 * pw - kw) // sw + 1
    batched = col.rank == 3
    c3 = col if batched else col.reshape(1, *col.shape)
    if c3.rank != 3 or c3.shape[1] != channels * kh * kw or c3.shape[2] != ho * wo:
        raise ValueError(f"col2im: column matrix of shape {col.shape} does not match the geometry")
    if c3.strides[2] != 1:
        c3 = c3.clone()
    N = c3.shape[0]
    out = empty((N, channels, height, width), col.dtype)
    check(getattr(_lib.load(), f"am_hip_col2im_{col.sfx}")(
        N, channels, height, width, kh, kw, ph, pw, sh, sw, ctypes.c_void_p(c3.data_ptr()), c3.strides[0], c3.strides[1],
        ctypes.c_void_p(out.data_ptr()), *out.strides))
    return out if batched else out.reshape(channels, height, width)


def conv2d_backward(input: HipTensor, weight: HipTensor, bias: HipTensor | None, padding, stride, grad_output: HipTensor,
                    need_input_grad: bool = True, fused_weight_gradient: bool = True):
    """(grad_input, grad_weight, grad_bias) of conv2d_backward (src/arraymancer/nn_primitives/nnp_convolution.nim:65-107)
    over im2colgemm_conv2d_gradient (fallback/conv.nim:107-145). The reference loops over the images (two GEMMs, an
    im2col and a col2im each); here the batch is folded into the columns, g[C_out, N*P] = grad_output with its first
    two axes swapped and col[C*kH*kW, N*P] the column matrices side by side, so that the whole pass is

        grad_bias   = row sums of g                      (sum(3).sum(2).sum(0) of the reference)
        grad_weight = g * col^T                          (one product with k = N*P; the per-image products summed)
        grad_input  = col2im(kernel_col^T * g)           (one product, one gather)

    Float tensors with unit stride and up to 96 input channels (float32: any number on images of 512 pixels or more)
    take grad_input as ONE launch instead: the convolution of grad_output with the turned kernel. Float tensors whose
    window steps by one pixel along the width, with output rows of whole 16-byte vectors, take grad_weight as ONE launch
    too: col^T is gathered from the images by the product's loader and never written (`fused_weight_gradient=False`:
    im2col + product as above; the same bits wherever both pick the same tile and split of k). grad_bias is None when `bias` is;
    grad_input is None (and not computed) when `need_input_grad` is False: the first layer of a network has no use for
    the gradient of the images."""
    _same_dtype(input, weight, grad_output)
    N, C, H, W = input.shape
    co, ci, kh, kw = weight.shape
    if ci != C:
        raise ValueError(f"conv2d_backward: kernel expects {ci} input channels, input has {C}")
    ho, wo = (H + 2 * padding[0] - kh) // stride[0] + 1, (W + 2 * padding[1] - kw) // stride[1] + 1
    if grad_output.shape != (N, co, ho, wo):
        raise ValueError(f"conv2d_backward: grad_output is {grad_output.shape}, the convolution's result is {(N, co, ho, wo)}")
    P = ho * wo
    g = grad_output.reshape(N, co, P).permute(1, 0, 2).clone().reshape(co, N * P)
    grad_bias = tsum(g, axis=1).reshape(*bias.shape) if bias is not None else None
    kcol = weight.reshape(co, ci * kh * kw)
    vk = 16 // input.dtype.itemsize
    if (fused_weight_gradient and input.dtype.kind == "f" and stride[1] == 1 and input.strides[3] == 1 and wo % vk == 0 and W >= vk
            and N >= 1 and P >= 1 and N * P < 2 ** 31 and ci * kh * kw * kh * kw < 2 ** 32 and co * ci * kh * kw < 1_000_000):
        # one launch: the product's second operand is gathered from the images, the column matrix (k^2 times the batch)
        # is neither written nor read back (float32 64 x 64 x 56 x 56, 3 x 3: 350 -> 257 us with the swap of grad_output).
        # A gradient of a million elements or more stays with the plain product and its larger tiles
        # (16 x 512 x 8 x 8 -> 512: 63 against 89 us).
        grad_weight = empty((co, ci, kh, kw), input.dtype)
        check(getattr(_lib.load(), f"am_hip_conv2d_grad_weight_{input.sfx}")(
            N, C, H, W, co, kh, kw, padding[0], padding[1], stride[0], stride[1], ctypes.c_void_p(input.data_ptr()), *input.strides,
            ctypes.c_void_p(g.data_ptr()), g.strides[0], ctypes.c_void_p(grad_weight.data_ptr())))
    else:
        col = im2col_folded(input, (kh, kw), padding, stride)
        grad_weight = matmul(g, col.transpose()).reshape(co, ci, kh, kw)
    if not need_input_grad:
        return None, grad_weight, grad_bias
    if (input.dtype.kind == "f" and tuple(stride) == (1, 1) and padding[0] < kh and padding[1] < kw and N <= 65535
            and (C <= 96 or (input.dtype == np.float32 and H * W >= 512))
            and co * kh * kw * input.dtype.itemsize >= 16):
        # With unit stride the gradient is itself a convolution, of grad_output with the kernel turned by 180 degrees and
        # its two channel axes swapped, padded by k - 1 - p: one launch of the gathered form instead of a product that
        # writes the column matrix of the gradient and a pass that reads it back (64 x 64 x 56 x 56, 3 x 3: 416 -> 191 us).
        turned = weight.permute(1, 0, 2, 3)[:, :, ::-1, ::-1].clone()
        grad_input = conv2d_into(empty((N, C, H, W), input.dtype), grad_output, turned, None, (kh - 1 - padding[0], kw - 1 - padding[1]))
        return grad_input, grad_weight, grad_bias
    gcol = matmul(kcol.transpose(), g)                      # [C*kH*kW, N*P]
    grad_input = empty((N, C, H, W), input.dtype)
    check(getattr(_lib.load(), f"am_hip_col2im_{input.sfx}")(
        N, C, H, W, kh, kw, padding[0], padding[1], stride[0], stride[1], ctypes.c_void_p(gcol.data_ptr()), P, N * P,
        ctypes.c_void_p(grad_input.data_ptr()), *grad_input.strides))
    return grad_input, grad_weight, grad_bias


def conv2d_into(out: HipTensor, x: HipTensor, kernel: HipTensor, bias: HipTensor | None = None, padding=(0, 0), stride=(1, 1),
                relu: bool = False) -> HipTensor:
    """The fused convolution of `conv2d` written into an existing C-contiguous [N, C_out, H_out, W_out] tensor: one
    launch, nothing allocated (what a captured graph needs). Float tensors, kernel rows with unit stride."""
    _same_dtype(x, kernel, out)
    N, C, H, W = x.shape
    co, ci, kh, kw = kernel.shape
    kcol = kernel.reshape(co, ci * kh * kw)
    if kcol.strides[1] != 1 or not out.is_C_contiguous():
        raise ValueError("conv2d_into: the kernel needs unit stride within a row and the result must be C-contiguous")
    epi = EPI[("bias_relu" if relu else "bias") if bias is not None else ("relu" if relu else "none")]
    bptr, bs = (ctypes.c_void_p(bias.data_ptr()), bias.reshape(co).strides[0]) if bias is not None else (None, 0)
    check(getattr(_lib.load(), f"am_hip_conv2d_{x.sfx}")(
        N, C, H, W, co, kh, kw, padding[0], padding[1], stride[0], stride[1], ctypes.c_void_p(x.data_ptr()), *x.strides,
        ctypes.c_void_p(kcol.data_ptr()), kcol.strides[0], epi, bptr, bs, ctypes.c_void_p(out.data_ptr())))
    return out


def conv2d(x: HipTensor, kernel: HipTensor, bias: HipTensor | None = None, padding=(0, 0), stride=(1, 1),
           relu: bool = False, fused: bool | None = None) -> HipTensor:
    """im2colgemm_conv2d (src/arraymancer/nn_primitives/fallback/conv.nim:81-106). Float tensors: ONE launch, a
    batched GEMM kernel_col[C_out, C*kH*kW] * col[n] whose B loader gathers the column matrix from the images
    (it is never written), with the bias [C_out, 1, 1] (and an optional ReLU) in its epilogue. Integer tensors, and
    `fused=False`: device im2col of the batch, then one strided-batched GEMM written straight into the NCHW result."""
    _same_dtype(x, kernel)
    N, C, H, W = x.shape
    co, ci, kh, kw = kernel.shape
    if ci != C:
        raise ValueError(f"conv2d: kernel expects {ci} input channels, input has {C}")
    ho, wo = (H + 2 * padding[0] - kh) // stride[0] + 1, (W + 2 * padding[1] - kw) // stride[1] + 1
    is_float = x.dtype.kind == "f"
    if fused is None:
        # up to about a hundred output channels the gathered form wins (no column matrix is written and read back);
        # beyond, the two-launch form's larger tiles catch up on small images (float32 32 x 256 x 14 x 14 -> 256, 3 x 3:
        # 130 against 95 us) but not on large ones (64 x 64 x 56 x 56 -> 128: 324 against 427 us; 28 x 28 is even)
        fused = (is_float and ci * kh * kw * x.dtype.itemsize >= 16 and N <= 65535
                 and (co <= 96 or (x.dtype == np.float32 and ho * wo >= 512)))
    if fused:
        k = kernel if kernel.reshape(co, ci * kh * kw).strides[1] == 1 else kernel.clone()
        return conv2d_into(empty((N, co, ho, wo), x.dtype), x, k, bias, padding, stride, relu)
    col = im2col(x, (kh, kw), padding, stride)
    out = empty((N, co, ho, wo), x.dtype)
    out3 = out.reshape(N, co, ho * wo)
    kcol = kernel.reshape(co, ci * kh * kw)
    if bias is not None and is_float:
        gemm_batched(1, kcol, col, 0, out3, epilogue="bias_relu" if relu else "bias", bias=bias.reshape(co, 1))
    else:
        gemm_batched(1, kcol, col, 0, out3, epilogue="relu" if (relu and is_float) else "none")
        if bias is not None:
            out3.bc_iadd(bias.reshape(1, co, 1))
        if relu and not is_float:
            _unary_into("relu", out3, out3)
    return out


def linear(x: HipTensor, weight: HipTensor, bias: HipTensor | None = None, relu: bool = False) -> HipTensor:
    """out = x * weight.transpose (+ bias) (then ReLU) in ONE kernel — the three passes of
    src/arraymancer/nn_primitives/nnp_linear.nim:20-29 + nnp_activation.nim:35-36 fused into the
    GEMM epilogue. weight is [out_features, in_features], bias [1, out_features]."""
    out = empty((x.shape[0], weight.shape[0]), x.dtype)
    epi = ("bias_relu" if relu else "bias") if bias is not None else ("relu" if relu else "none")
    return gemm(1, x, weight.transpose(), 0, out, epilogue=epi, bias=bias)


def linear_backward(input: HipTensor, weight: HipTensor, gradOutput: HipTensor, with_bias: bool = True):
    """(gradInput, gradWeight[, gradBias]) of src/arraymancer/nn_primitives/nnp_linear.nim:39-66:
    gradInput = gradOutput * weight, gradWeight = gradOutput.transpose * input (the transposed
    view goes to the GEMM as strides), gradBias = sum(gradOutput, axis=0) of shape
    [1, out_features]."""
    grad_input = matmul(gradOutput, weight)
    grad_weight = matmul(gradOutput.transpose(), input)
    if not with_bias:
        return grad_input, grad_weight
    return grad_input, grad_weight, tsum(gradOutput, axis=0)


# ---------------------------------------------------------------------- optimizer
def sgd_update(values, gradients, learning_rate: float):
    """value -= learning_rate * gradient for every (value, gradient) pair in ONE launch: the update of the SGD optimizer
    (src/arraymancer/nn/optimizers/optimizers.nim:35-51 runs one apply2_inline per parameter). C-contiguous float
    tensors of one element type; each gradient has its value's shape."""
    values, gradients = list(values), list(gradients)
    if len(values) != len(gradients):
        raise ValueError("sgd_update: one gradient per value")
    if not values:
        return
    _same_dtype(*values, *gradients)
    if values[0].dtype.kind != "f":
        raise TypeError("sgd_update is defined for float tensors")
    for v, g in zip(values, gradients):
        if v.shape != g.shape:
            raise ValueError(f"sgd_update: gradient of shape {g.shape} for a value of shape {v.shape}")
        if not (v.is_C_contiguous() and g.is_C_contiguous()):
            raise ValueError("sgd_update: values and gradients must be C-contiguous")
    n = len(values)
    ptrs = lambda ts: (ctypes.c_void_p * n)(*[t.data_ptr() for t in ts])
    check(getattr(_lib.load(), f"am_hip_sgd_update_{values[0].sfx}")(
        n, ptrs(values), ptrs(gradients), i64_array([v.size for v in values]), _lib.CTYPE[values[0].sfx](learning_rate)))


# ---------------------------------------------------------------------- gated recurrent unit
def _gru_gates_inplace(W3x: HipTensor, U3h: HipTensor, hidden: HipTensor, keep=None):
    """Steps 2-4 of gru_cell_inference / gru_cell_forward (nnp_gru.nim:72-88, 125-146) as one launch over the two
    [batch, 3H] products; `hidden` is updated in place. keep = (r, z, n, Uh) receives what the backward pass needs."""
    B, H = hidden.shape
    if W3x.shape != (B, 3 * H) or U3h.shape != (B, 3 * H):
        raise ValueError(f"gru: products of shape {W3x.shape} and {U3h.shape} for a hidden state {hidden.shape}")
    if W3x.strides[1] != 1 or U3h.strides[1] != 1 or hidden.strides[1] != 1:
        raise ValueError("gru: the rows of the products and of the hidden state need unit stride")
    saved = [ctypes.c_void_p(t.data_ptr()) for t in keep] if keep else [None] * 4
    lds = keep[0].strides[0] if keep else 0
    if keep and any(t.shape != (B, H) or t.strides != keep[0].strides or t.strides[1] != 1 for t in keep):
        raise ValueError("gru: r, z, n and Uh must be [batch, H] tensors of one layout")
    check(getattr(_lib.load(), f"am_hip_gru_gates_{hidden.sfx}")(
        B, H, ctypes.c_void_p(W3x.data_ptr()), W3x.strides[0], ctypes.c_void_p(U3h.data_ptr()), U3h.strides[0],
        ctypes.c_void_p(hidden.data_ptr()), hidden.strides[0], *saved, lds))


def gru_cell_inference(input: HipTensor, W3: HipTensor, U3: HipTensor, bW3: HipTensor, bU3: HipTensor, hidden: HipTensor) -> HipTensor:
    """gru_cell_inference (src/arraymancer/nn_primitives/nnp_gru.nim:40-88): h(t) -> h'(t) in place. Two dense layers
    with the bias in the GEMM epilogue ([batch, 3H] each), then the gate arithmetic (sigmoid(x + y) for the reset and update
    gates, tanh(x + r * u) for the candidate, (1 - z) * n + z * h into `hidden`) as one launch.
    input [batch, features], W3 [3H, features], U3 [3H, H], biases [1, 3H]."""
    _gru_gates_inplace(linear(input, W3, bW3), linear(hidden, U3, bU3), hidden)
    return hidden


def gru_cell_forward(input: HipTensor, W3: HipTensor, U3: HipTensor, bW3: HipTensor, bU3: HipTensor, hidden: HipTensor):
    """gru_cell_forward (nnp_gru.nim:90-146): like gru_cell_inference, keeping what the backward pass needs. Updates
    `hidden` in place and returns (r, z, n, Uh), each [batch, H]."""
    B, H = hidden.shape
    keep = tuple(empty((B, H), hidden.dtype) for _ in range(4))
    _gru_gates_inplace(linear(input, W3, bW3), linear(hidden, U3, bU3), hidden, keep)
    return keep


def _gru_gates_backward_passes(dnext, h, r, z, n, Uh, dW3x, dU3h):
    """The element-wise part of gru_cell_backward (nnp_gru.nim:165-186) with the reference's separate bodies, written
    into column slices of the two [batch, 3H] buffers where the reference concatenates. Nine launches; kept as the
    statement the one-launch kernel is compared with."""
    H = h.shape[1]
    sr, sz, s_ = slice(0, H), slice(H, 2 * H), slice(2 * H, 3 * H)
    dz = map2("mul", map2("sub", h, n), dnext)                                   # step 4, z part
    dn = map2("mul", scalar_op("sub", z, 1, scalar_on_left=True), dnext)
    _binary_into("tanh_bwd", dW3x[:, s_], n, dn)                                 # step 3: dWx = dn * (1 - n * n)
    dr = map2("mul", Uh, dW3x[:, s_])
    _binary_into("mul", dU3h[:, s_], r, dW3x[:, s_])                             # dUh = r * dWx
    _binary_into("sigmoid_bwd", dW3x[:, sz], z, dz)                              # step 2: update gate
    _binary_into("sigmoid_bwd", dW3x[:, sr], r, dr)                              # step 2: reset gate
    _unary_into("copy", dU3h[:, 0:2 * H], dW3x[:, 0:2 * H])                      # dUrh = dWrx, dUzh = dWzx


def gru_cell_backward(dnext: HipTensor, x: HipTensor, h: HipTensor, W3: HipTensor, U3: HipTensor,
                      r: HipTensor, z: HipTensor, n: HipTensor, Uh: HipTensor):
    """gru_cell_backward (nnp_gru.nim:148-192): (dx, dh, dW3, dU3, dbW3, dbU3) from the gradient `dnext` of the next
    hidden state, the inputs of the forward pass (h is the hidden state BEFORE it) and the tensors it saved. The
    element-wise steps and the two concatenations of the reference are one launch that writes the gate gradients into
    the column slices of one [batch, 3H] buffer per dense layer; then the two linear_backward and dh + dnext * z."""
    B, H = h.shape
    dW3x, dU3h = empty((B, 3 * H), h.dtype), empty((B, 3 * H), h.dtype)
    saved = (dnext, h, r, z, n, Uh)
    same = all(t.shape == (B, H) and t.strides == dnext.strides and t.strides[1] == 1 for t in saved)
    if same:
        check(getattr(_lib.load(), f"am_hip_gru_gates_backward_{h.sfx}")(
            B, H, *[ctypes.c_void_p(t.data_ptr()) for t in saved], dnext.strides[0],
            ctypes.c_void_p(dW3x.data_ptr()), 3 * H, ctypes.c_void_p(dU3h.data_ptr()), 3 * H))
    else:   # operands of different layouts: the separate passes take any strides
        _gru_gates_backward_passes(dnext, h, r, z, n, Uh, dW3x, dU3h)
    dx, dW3, dbW3 = linear_backward(x, W3, dW3x)                                 # step 1
    dh, dU3, dbU3 = linear_backward(h, U3, dU3h)
    _ternary_into("muladd", dh, dnext, z, dh)                                    # step 4, h part: dh + dnext * z
    return dx, dh, dW3, dU3, dbW3, dbU3


def gru_inference(input: HipTensor, W3s0: HipTensor, W3sN: HipTensor | None, U3s: HipTensor, bW3s: HipTensor, bU3s: HipTensor,
                  hidden: HipTensor) -> HipTensor:
    """gru_inference (nnp_gru.nim:194-262): a stack of GRU layers over a sequence. input [timesteps, batch, features];
    W3s0 [3H, features]; W3sN [layers - 1, 3H, H] (None or empty for one layer); U3s [layers, 3H, H]; biases
    [layers, 1, 3H]; hidden [layers, batch, H], updated in place to the state after the last timestep. Returns the
    output [timesteps, batch, H]: the top layer's hidden state at every timestep."""
    T, B, F = input.shape
    H = hidden.shape[2]
    layers = 1 + (W3sN.shape[0] if W3sN is not None and W3sN.size else 0)
    if hidden.shape != (layers, B, H) or W3s0.shape != (3 * H, F) or U3s.shape != (layers, 3 * H, H) or \
            bW3s.shape != (layers, 1, 3 * H) or bU3s.shape != bW3s.shape or (layers > 1 and W3sN.shape != (layers - 1, 3 * H, H)):
        raise ValueError("gru_inference: shapes of the weights, biases and hidden state do not fit the input")
    output = empty((T, B, H), input.dtype)
    for layer in range(layers):
        W3l = W3s0 if layer == 0 else W3sN[layer - 1].squeeze(0)
        U3l, bW3l, bU3l, h_l = U3s[layer].squeeze(0), bW3s[layer].squeeze(0), bU3s[layer].squeeze(0), hidden[layer].squeeze(0)
        # The input side of the layer does not depend on the recurrence: W3 * x + bW3 for ALL timesteps is one product
        # [T * batch, features] * W3^T (the reference multiplies per timestep; row by row the same dot products).
        src = input if layer == 0 else output
        W3x_all = linear(src.reshape(T * B, src.shape[2]), W3l, bW3l).reshape(T, B, 3 * H)
        for t in range(T):
            _gru_gates_inplace(W3x_all[t].squeeze(0), linear(h_l, U3l, bU3l), h_l)
            _unary_into("copy", output[t].squeeze(0), h_l)
    return output


def _gru_layer_weights(layer, W3s0, W3sN, U3s, bW3s=None, bU3s=None):
    W3l = W3s0 if layer == 0 else W3sN[layer - 1].squeeze(0)
    out = [W3l, U3s[layer].squeeze(0)]
    if bW3s is not None:
        out += [bW3s[layer].squeeze(0), bU3s[layer].squeeze(0)]
    return out


def gru_forward(input: HipTensor, W3s0: HipTensor, W3sN: HipTensor | None, U3s: HipTensor, bW3s: HipTensor, bU3s: HipTensor,
                hidden: HipTensor):
    """gru_forward (nnp_gru.nim:263-374): gru_inference that keeps what gru_backward needs. Returns (output, cache);
    `hidden` [layers, batch, H] is updated in place. The cache holds, per layer, the layer's input [T, batch, features]
    and, time-major [T, batch, H], the hidden state before every step and the r, z, n, Uh of every step (the reference
    keeps the same values as seq[Tensor] / [layers, T, batch, H] tensors)."""
    T, B, F = input.shape
    H = hidden.shape[2]
    layers = 1 + (W3sN.shape[0] if W3sN is not None and W3sN.size else 0)
    if hidden.shape != (layers, B, H) or W3s0.shape != (3 * H, F) or U3s.shape != (layers, 3 * H, H) or \
            bW3s.shape != (layers, 1, 3 * H) or bU3s.shape != bW3s.shape or (layers > 1 and W3sN.shape != (layers - 1, 3 * H, H)):
        raise ValueError("gru_forward: shapes of the weights, biases and hidden state do not fit the input")
    output = empty((T, B, H), input.dtype)
    cache = []
    for layer in range(layers):
        W3l, U3l, bW3l, bU3l = _gru_layer_weights(layer, W3s0, W3sN, U3s, bW3s, bU3s)
        src = input if layer == 0 else output.clone()
        W3x_all = linear(src.reshape(T * B, src.shape[2]), W3l, bW3l).reshape(T, B, 3 * H)
        h_l = hidden[layer].squeeze(0)
        hs, r, z, n, Uh = (empty((T, B, H), input.dtype) for _ in range(5))
        for t in range(T):
            _unary_into("copy", hs[t].squeeze(0), h_l)
            keep = tuple(a[t].squeeze(0) for a in (r, z, n, Uh))
            _gru_gates_inplace(W3x_all[t].squeeze(0), linear(h_l, U3l, bU3l), h_l, keep)
            _unary_into("copy", output[t].squeeze(0), h_l)
        cache.append(dict(input=src, hiddens=hs, r=r, z=z, n=n, Uh=Uh))
    return output, cache


def gru_backward(dOutput: HipTensor, dHiddenN: HipTensor, cache, W3s0: HipTensor, W3sN: HipTensor | None, U3s: HipTensor):
    """gru_backward (nnp_gru.nim:376-500): (dInput, dHidden0, dW3s0, dW3sN, dU3s, dbW3s, dbU3s) from the gradients of the
    output [T, batch, H] and of the last hidden state [layers, batch, H]. Only the recurrence is walked step by step
    (per step the one-launch gate gradients, one product with U3 and dh + dnext * z); the gradients of the weights, biases
    and of the layer's input are taken over all timesteps at once afterwards - four products and two column sums per
    layer where the reference accumulates four products per step (the same sums in another order)."""
    layers = len(cache)
    T, B, H = cache[0]["r"].shape
    dt = dOutput.dtype
    if dOutput.shape != (T, B, H) or dHiddenN.shape != (layers, B, H):
        raise ValueError("gru_backward: gradients of shape [T, batch, H] and [layers, batch, H] expected")
    gflow = dOutput.clone()
    dHidden0 = empty((layers, B, H), dt)
    dW3sN = empty(W3sN.shape, dt) if layers > 1 else None
    dU3s, dbW3s, dbU3s = empty(U3s.shape, dt), empty((layers, 1, 3 * H), dt), empty((layers, 1, 3 * H), dt)
    dInput = dW3s0 = None
    for layer in range(layers - 1, -1, -1):
        W3l, U3l = _gru_layer_weights(layer, W3s0, W3sN, U3s)
        c = cache[layer]
        dW3x_all, dU3h_all = empty((T, B, 3 * H), dt), empty((T, B, 3 * H), dt)
        dht1 = dHiddenN[layer].squeeze(0).clone()
        for t in range(T - 1, -1, -1):
            apply2("add", dht1, gflow[t].squeeze(0))
            saved = (dht1,) + tuple(c[k][t].squeeze(0) for k in ("hiddens", "r", "z", "n", "Uh"))
            check(getattr(_lib.load(), f"am_hip_gru_gates_backward_{saved[0].sfx}")(
                B, H, *[ctypes.c_void_p(a.data_ptr()) for a in saved], H,
                ctypes.c_void_p(dW3x_all[t].data_ptr()), 3 * H, ctypes.c_void_p(dU3h_all[t].data_ptr()), 3 * H))
            dh = matmul(dU3h_all[t].squeeze(0), U3l)
            _ternary_into("muladd", dh, dht1, c["z"][t].squeeze(0), dh)
            dht1 = dh
        _unary_into("copy", dHidden0[layer].squeeze(0), dht1)
        X = c["input"].reshape(T * B, c["input"].shape[2])
        G, GU = dW3x_all.reshape(T * B, 3 * H), dU3h_all.reshape(T * B, 3 * H)
        dx_all = matmul(G, W3l)
        dW3 = matmul(G.transpose(), X)
        if layer == 0:
            dInput, dW3s0 = dx_all.reshape(T, B, X.shape[1]), dW3
        else:
            gflow = dx_all.reshape(T, B, H)
            _unary_into("copy", dW3sN[layer - 1].squeeze(0), dW3)
        gemm(1, GU.transpose(), c["hiddens"].reshape(T * B, H), 0, dU3s[layer].squeeze(0))
        reduce_axis_into("sum", dbW3s[layer].squeeze(0), G, 0)
        reduce_axis_into("sum", dbU3s[layer].squeeze(0), GU, 0)
    return dInput, dHidden0, dW3s0, dW3sN, dU3s, dbW3s, dbU3s


# ---------------------------------------------------------------------- element-wise
def _binary_into(op, dst: HipTensor, a: HipTensor, b: HipTensor):
    sfx = dst.ring_sfx if op in _RING_OPS else dst.sfx
    code = OP[op] if isinstance(op, str) else int(op)
    check(getattr(_lib.load(), f"am_hip_ew_binary_{sfx}")(
        code, dst.rank, i64_array(dst.shape),
        ctypes.c_void_p(dst.data_ptr()), i64_array(dst.strides),
        ctypes.c_void_p(a.data_ptr()), i64_array(a.strides),
        ctypes.c_void_p(b.data_ptr()), i64_array(b.strides)))


def _scalar_into(op, dst: HipTensor, a: HipTensor, scalar, left: bool):
    sfx = dst.ring_sfx if op in _RING_OPS else dst.sfx
    code = OP[op] if isinstance(op, str) else int(op)
    check(getattr(_lib.load(), f"am_hip_ew_scalar_{sfx}")(
        code, int(bool(left)), dst.rank, i64_array(dst.shape),
        ctypes.c_void_p(dst.data_ptr()), i64_array(dst.strides),
        ctypes.c_void_p(a.data_ptr()), i64_array(a.strides),
        _ring_scalar(sfx, dst.dtype, scalar) if dst.dtype in _UNSIGNED_TWIN else CTYPE[sfx](scalar)))


def _unary_into(op, dst: HipTensor, a: HipTensor):
    sfx = dst.ring_sfx if op in _RING_UOPS else dst.sfx
    code = UOP[op] if isinstance(op, str) else int(op)
    check(getattr(_lib.load(), f"am_hip_ew_unary_{sfx}")(
        code, dst.rank, i64_array(dst.shape),
        ctypes.c_void_p(dst.data_ptr()), i64_array(dst.strides),
        ctypes.c_void_p(a.data_ptr()), i64_array(a.strides)))


def map2(op, a: HipTensor, b: HipTensor) -> HipTensor:
    """map2_inline with one of the enumerated bodies: fresh C-contiguous result; operands must
    already have equal shapes (src/arraymancer/tensor/higher_order_applymap.nim:92-120)."""
    _same_dtype(a, b)
    _check_elementwise(a, b)
    _ = a.ring_sfx if op in _RING_OPS else a.sfx      # (refuses before anything is allocated)
    if op in CMP:   # a body with a bool result: the output type follows the body, like the reference's template
        out = empty(a.shape, np.bool_)
        if out.size:
            _compare_into(op, out, a, b)
        return out
    out = empty(a.shape, a.dtype)
    _binary_into(op, out, a, b)
    return out


def apply2(op, dest: HipTensor, src: HipTensor) -> HipTensor:
    """apply2_inline: dest[i] = op(dest[i], src[i]) through dest's own strides (:40-47)."""
    _same_dtype(dest, src)
    _check_elementwise(dest, src)
    _binary_into(op, dest, dest, src)
    return dest


def _compare_into(cmp, dst: HipTensor, a: HipTensor, b: HipTensor):
    check(getattr(_lib.load(), f"am_hip_ew_compare_{a.sfx}")(
        CMP[cmp], dst.rank, i64_array(dst.shape), ctypes.c_void_p(dst.data_ptr()), i64_array(dst.strides),
        ctypes.c_void_p(a.data_ptr()), i64_array(a.strides), ctypes.c_void_p(b.data_ptr()), i64_array(b.strides)))


def _ternary_into(op, dst: HipTensor, a: HipTensor, b: HipTensor, c: HipTensor):
    code = OP3[op] if isinstance(op, str) else int(op)
    check(getattr(_lib.load(), f"am_hip_ew_ternary_{dst.ring_sfx if op in _RING_OP3 else dst.sfx}")(
        code, dst.rank, i64_array(dst.shape), ctypes.c_void_p(dst.data_ptr()), i64_array(dst.strides),
        ctypes.c_void_p(a.data_ptr()), i64_array(a.strides), ctypes.c_void_p(b.data_ptr()), i64_array(b.strides),
        ctypes.c_void_p(c.data_ptr()), i64_array(c.strides)))


def map3(op, a: HipTensor, b: HipTensor, c: HipTensor) -> HipTensor:
    """map3_inline with an enumerated body ("muladd": x*y+z, "gru_candidate": tanh(x+y*z),
    "gru_blend": (1-y)*z+y*x); src/arraymancer/tensor/higher_order_applymap.nim:122-150."""
    _same_dtype(a, b, c)
    _check_elementwise(a, b)
    _check_elementwise(a, c)
    _ = a.ring_sfx if op in _RING_OP3 else a.sfx
    out = empty(a.shape, a.dtype)
    if out.size:
        _ternary_into(op, out, a, b, c)
    return out


def apply3(op, dest: HipTensor, src1: HipTensor, src2: HipTensor) -> HipTensor:
    """apply3_inline: dest[i] = op(dest[i], src1[i], src2[i]) through dest's own strides (:58-67)."""
    _same_dtype(dest, src1, src2)
    _check_elementwise(dest, src1)
    _check_elementwise(dest, src2)
    if dest.size:
        _ternary_into(op, dest, dest, src1, src2)
    return dest


def _bc(op, a: HipTensor, b: HipTensor) -> HipTensor:
    _same_dtype(a, b)
    la, lb = md.broadcast2(a.layout, b.layout)
    return map2(op, HipTensor(la, a.storage, a.dtype), HipTensor(lb, b.storage, b.dtype))


def bc_add(a, b): return _bc_or_scalar("add", a, b)
def bc_sub(a, b): return _bc_or_scalar("sub", a, b)
def bc_mul(a, b): return _bc_or_scalar("mul", a, b)
def bc_div(a, b): return _bc_or_scalar("div", a, b)
def bc_mod(a, b): return _bc_or_scalar("mod", a, b)


def floorMod(a, b):
    """floorMod(tensor, tensor) (equal shapes: map2_inline without broadcasting), floorMod(tensor, scalar),
    floorMod(scalar, tensor) (src/arraymancer/tensor/math_functions.nim:134-144)."""
    ta, tb = isinstance(a, HipTensor), isinstance(b, HipTensor)
    if ta and tb:
        return map2("floormod", a, b)
    return _bc_or_scalar("floormod", a, b)


def copySign(t1: HipTensor, t2: HipTensor) -> HipTensor:
    """Magnitudes of t1 with the signs of t2, float tensors (math_functions.nim:119-125)."""
    if t1.dtype.kind != "f":
        raise TypeError("copySign is defined for float tensors only")
    return map2("copysign", t1, t2)


def mcopySign(t1: HipTensor, t2: HipTensor) -> HipTensor:
    """In-place copySign (math_functions.nim:127-132)."""
    if t1.dtype.kind != "f":
        raise TypeError("mcopySign is defined for float tensors only")
    return apply2("copysign", t1, t2)


# ---- comparisons: `==.` `!=.` `<.` `<=.` `>.` `>=.` (src/arraymancer/tensor/operators_comparison.nim:41-185)
_MIRROR = {"==": "==", "!=": "!=", "<": ">", "<=": ">=", ">": "<", ">=": "<="}


def _bc_compare(cmp, a, b) -> HipTensor:
    """Tensor-tensor with implicit broadcasting, tensor-scalar, or scalar-tensor (which the reference
    rewrites into the mirrored tensor-scalar comparison, :150-185). Result: a bool tensor."""
    ta, tb = isinstance(a, HipTensor), isinstance(b, HipTensor)
    if ta and tb:
        _same_dtype(a, b)
        la, lb = md.broadcast2(a.layout, b.layout)
        return map2(cmp, HipTensor(la, a.storage, a.dtype), HipTensor(lb, b.storage, b.dtype))
    if not (ta or tb):
        raise TypeError("at least one operand must be a HipTensor")
    t, value, cmp = (a, b, cmp) if ta else (b, a, _MIRROR[cmp])
    _ = t.sfx
    out = empty(t.shape, np.bool_)      # returnEmptyIfEmpty: an empty tensor comes back empty
    if out.size:
        check(getattr(_lib.load(), f"am_hip_ew_compare_scalar_{t.sfx}")(
            CMP[cmp], out.rank, i64_array(out.shape), ctypes.c_void_p(out.data_ptr()), i64_array(out.strides),
            ctypes.c_void_p(t.data_ptr()), i64_array(t.strides), CTYPE[t.sfx](value)))
    return out


def bc_eq(a, b): return _bc_compare("==", a, b)
def bc_ne(a, b): return _bc_compare("!=", a, b)
def bc_lt(a, b): return _bc_compare("<", a, b)
def bc_le(a, b): return _bc_compare("<=", a, b)
def bc_gt(a, b): return _bc_compare(">", a, b)
def bc_ge(a, b): return _bc_compare(">=", a, b)


def _predicate(op, t: HipTensor, out_dtype) -> HipTensor:
    if t.dtype.kind != "f":
        raise TypeError(f"{op} is defined for float tensors only")
    out = empty(t.shape, out_dtype)
    if out.size:
        check(getattr(_lib.load(), f"am_hip_ew_predicate_{t.sfx}")(
            PRED[op], out.rank, i64_array(out.shape), ctypes.c_void_p(out.data_ptr()), i64_array(out.strides),
            ctypes.c_void_p(t.data_ptr()), i64_array(t.strides)))
    return out


def isNaN(t: HipTensor) -> HipTensor:
    """Bool tensor, true where x != x (operators_comparison.nim:192-198)."""
    return _predicate("isnan", t, np.bool_)


def isNotNaN(t: HipTensor) -> HipTensor:
    """Bool tensor, true where x == x (operators_comparison.nim:200-206)."""
    return _predicate("isnotnan", t, np.bool_)


# Ordinals of Nim's FloatClass, the element type of classify's result (math_functions.nim:264-276).
FLOAT_CLASS = ("fcNormal", "fcSubnormal", "fcZero", "fcNegZero", "fcNan", "fcInf", "fcNegInf")


def classify(t: HipTensor) -> HipTensor:
    """uint8 tensor of FloatClass ordinals (index into FLOAT_CLASS)."""
    return _predicate("classify", t, np.uint8)


def sgn(t: HipTensor) -> HipTensor:
    """int64 tensor (the reference's Tensor[int]) of -1 / 0 / 1; zeros and NaN give 0
    (src/arraymancer/tensor/math_functions.nim:110-117)."""
    _ = t.sfx
    out = empty(t.shape, np.int64)
    if out.size:
        check(getattr(_lib.load(), f"am_hip_ew_sgn_{t.sfx}")(
            out.rank, i64_array(out.shape), ctypes.c_void_p(out.data_ptr()), i64_array(out.strides),
            ctypes.c_void_p(t.data_ptr()), i64_array(t.strides)))
    return out


def bc_pow(a, b):
    """`^.`: tensor ^. scalar = pow(x, exponent), scalar ^. tensor = pow(base, x); float tensors
    only, one operand a scalar (src/arraymancer/tensor/operators_broadcasted.nim:153-161)."""
    ta, tb = isinstance(a, HipTensor), isinstance(b, HipTensor)
    if ta == tb:
        raise TypeError("`^.` takes one tensor and one scalar")
    t, s = (a, b) if ta else (b, a)
    _float_scalar("^.", t, s)
    return scalar_op("pow", t, s, scalar_on_left=tb)


def _float_scalar(name, t: HipTensor, scalar):
    if t.dtype.kind != "f":
        raise TypeError(f"{name} is defined for float tensors only")
    if isinstance(scalar, HipTensor):
        raise TypeError(f"{name} takes a scalar")


def _bc_or_scalar(op, a, b):
    """`+.` and friends: tensor-tensor with implicit broadcasting, tensor-scalar, scalar-tensor
    (src/arraymancer/tensor/operators_broadcasted.nim:28-60, 107-161)."""
    ta, tb = isinstance(a, HipTensor), isinstance(b, HipTensor)
    if ta and tb:
        return _bc(op, a, b)
    if ta:
        return scalar_op(op, a, b)
    if tb:
        return scalar_op(op, b, a, scalar_on_left=True)
    raise TypeError("at least one operand must be a HipTensor")


def _bc_inplace(op, a: HipTensor, b):
    if not isinstance(b, HipTensor):
        _scalar_into(op, a, a, b, False)
        return a
    _same_dtype(a, b)
    bb = b.broadcast(a.shape)
    _binary_into(op, a, a, bb)
    return a


def scalar_op(op, t: HipTensor, scalar, scalar_on_left: bool = False) -> HipTensor:
    _ = t.ring_sfx if op in _RING_OPS else t.sfx
    out = empty(t.shape, t.dtype)
    if t.size:
        _scalar_into(op, out, t, scalar, scalar_on_left)
    return out


def unary(op, t: HipTensor) -> HipTensor:
    _ = t.ring_sfx if op in _RING_UOPS else t.sfx
    out = empty(t.shape, t.dtype)
    if t.size:
        _unary_into(op, out, t)
    return out


def relu(t: HipTensor) -> HipTensor:
    """src/arraymancer/nn_primitives/nnp_activation.nim:35-36."""
    return unary("relu", t)


def sigmoid(t: HipTensor) -> HipTensor:
    return unary("sigmoid", t)


def bias_relu(x: HipTensor, b: HipTensor) -> HipTensor:
    """map2_inline(x, b.broadcast(x.shape), max(0, x + y)) in one pass."""
    return _bc("add_relu", x, b)


def tanh(t: HipTensor) -> HipTensor:
    """src/arraymancer/nn_primitives/nnp_activation.nim:38-39."""
    return unary("tanh", t)


def relu_backward(gradient: HipTensor, cached_tensor: HipTensor) -> HipTensor:
    """map2_inline(cached_tensor, gradient): if x <= 0: 0 else: y
    (src/arraymancer/nn_primitives/nnp_activation.nim:65-70)."""
    return map2("relu_bwd", cached_tensor, gradient)


def sigmoid_backward(gradient: HipTensor, cached_tensor: HipTensor) -> HipTensor:
    """map2_inline(cached_tensor, gradient): x * (1 - x) * y (nnp_activation.nim:61-63)."""
    return map2("sigmoid_bwd", cached_tensor, gradient)


def tanh_backward(gradient: HipTensor, cached_tensor: HipTensor) -> HipTensor:
    """map2_inline(cached_tensor, gradient): y * (1 - x * x) (nnp_activation.nim:72-74)."""
    return map2("tanh_bwd", cached_tensor, gradient)


OPERATORS = {"+.": bc_add, "-.": bc_sub, "*.": bc_mul, "/.": bc_div, "mod": bc_mod,
             "^.": bc_pow,
             "==.": bc_eq, "!=.": bc_ne, "<.": bc_lt, "<=.": bc_le, ">.": bc_gt, ">=.": bc_ge,
             "+.=": HipTensor.bc_iadd, "-.=": HipTensor.bc_isub, "*.=": HipTensor.bc_imul,
             "/.=": HipTensor.bc_idiv, "^.=": HipTensor.bc_ipow}


# The universal functions of src/arraymancer/tensor/ufunc.nim:82-130 (makeUniversal: map_inline of
# the math library's function of the same name) and reciprocal (math_functions.nim:52-58).
UFUNCS = ("ln", "log10", "log2", "exp", "sqrt", "cbrt", "sin", "cos", "tan", "sinh", "cosh", "tanh",
          "arcsin", "arccos", "arctan", "arcsinh", "arccosh", "arctanh", "erf", "erfc", "gamma", "lgamma",
          "floor", "ceil", "trunc", "round", "reciprocal")


def _make_ufunc(name):
    def f(t: HipTensor) -> HipTensor:
        if t.dtype.kind != "f":
            raise TypeError(f"{name} is defined for float tensors only")
        return unary(name, t)
    f.__name__ = name
    f.__doc__ = f"Element-wise {name} of a float tensor (src/arraymancer/tensor/ufunc.nim:56-130)."
    return f


ln, log10, log2, exp, cbrt, sin, cos, tan, sinh, cosh, arcsin, arccos, arctan, arcsinh, arccosh, arctanh, \
    erf, erfc, gamma, lgamma, floor, ceil, trunc, reciprocal = (_make_ufunc(n) for n in (
        "ln", "log10", "log2", "exp", "cbrt", "sin", "cos", "tan", "sinh", "cosh", "arcsin", "arccos", "arctan",
        "arcsinh", "arccosh", "arctanh", "erf", "erfc", "gamma", "lgamma", "floor", "ceil", "trunc", "reciprocal"))
tround = _make_ufunc("round")


def degToRad(t: HipTensor) -> HipTensor:
    """x * (PI / 180) (src/arraymancer/tensor/ufunc.nim:129)."""
    if t.dtype.kind != "f":
        raise TypeError("degToRad is defined for float tensors only")
    return unary("degtorad", t)


def radToDeg(t: HipTensor) -> HipTensor:
    """x / (PI / 180) (src/arraymancer/tensor/ufunc.nim:130)."""
    if t.dtype.kind != "f":
        raise TypeError("radToDeg is defined for float tensors only")
    return unary("radtodeg", t)


def fac(t: HipTensor) -> HipTensor:
    """The factorial of every element (src/arraymancer/tensor/ufunc.nim:84-85 maps Nim's `fac`, a table of 0! .. 20!
    that asserts its argument lies inside it): integer tensors, every element in 0 .. 20, else ValueError
    (the range is checked with two reductions before the pass)."""
    if t.dtype.kind != "i":
        raise TypeError("fac is defined for integer tensors only")
    if t.size and (int(reduce_all("min", t)) < 0 or int(reduce_all("max", t)) > 20):
        raise ValueError("fac: every element must be a non-negative integer of at most 20")
    return unary("fac", t)


def _clamp_into(dst: HipTensor, t: HipTensor, lo, hi):
    # both bounds travel by value: no device allocation, no copy, no synchronisation, recordable into a graph
    ct = CTYPE[t.sfx]
    check(getattr(_lib.load(), f"am_hip_ew_clamp_{t.sfx}")(
        dst.rank, i64_array(dst.shape), ctypes.c_void_p(dst.data_ptr()), i64_array(dst.strides),
        ctypes.c_void_p(t.data_ptr()), i64_array(t.strides), ct(lo), ct(hi)))


def clamp(t: HipTensor, min, max) -> HipTensor:
    """map_inline(clamp(x, min, max)): min where x < min, max where x > max, else x
    (src/arraymancer/tensor/math_functions.nim:146-148). One pass."""
    _ = t.sfx
    out = empty(t.shape, t.dtype)
    if out.size:
        _clamp_into(out, t, min, max)
    return out


def mclamp(t: HipTensor, min, max) -> HipTensor:
    """In-place clamp (math_functions.nim:150-152)."""
    if t.size:
        _clamp_into(t, t, min, max)
    return t


def mreciprocal(t: HipTensor) -> HipTensor:
    """In-place 1 / x (src/arraymancer/tensor/math_functions.nim:56-58)."""
    if t.dtype.kind != "f":
        raise TypeError("mreciprocal is defined for float tensors only")
    if t.size:
        _unary_into("reciprocal", t, t)
    return t


# ---------------------------------------------------------------- reductions, softmax, pooling
def reduce_axis(op, t: HipTensor, axis: int) -> HipTensor:
    """reduce_axis_inline (src/arraymancer/tensor/higher_order_foldreduce.nim:46-61): fold along
    `axis`; the result keeps that axis with extent 1. An empty tensor comes back empty
    (returnEmptyIfEmpty, aggregate.nim:40); an axis outside the rank raises IndexError."""
    if not 0 <= axis < t.rank:
        raise IndexError(f"Input tensor rank ({t.rank}) must be greater than reduction axis ({axis})")
    _ = t.ring_sfx if op in _RING_RED else t.sfx
    if t.size == 0:
        return empty(t.shape, t.dtype)
    shape = list(t.shape)
    shape[axis] = 1
    return reduce_axis_into(op, empty(shape, t.dtype), t, axis)


def reduce_axis_into(op, out: HipTensor, t: HipTensor, axis: int) -> HipTensor:
    """reduce_axis written into an existing tensor of t's shape with extent 1 along `axis` (any strides): nothing is
    allocated, which a captured graph or a tight loop needs."""
    _same_dtype(out, t)
    if out.rank != t.rank or any(o != (1 if d == axis else n) for d, (o, n) in enumerate(zip(out.shape, t.shape))):
        raise ValueError(f"reduce_axis_into: result {out.shape} does not fit {t.shape} folded along axis {axis}")
    check(getattr(_lib.load(), f"am_hip_reduce_axis_{t.ring_sfx if op in _RING_RED else t.sfx}")(
        RED[op], t.rank, i64_array(t.shape), axis, ctypes.c_void_p(out.data_ptr()), i64_array(out.strides),
        ctypes.c_void_p(t.data_ptr()), i64_array(t.strides)))
    return out


def _argreduce(op, t: HipTensor, axis: int):
    if not 0 <= axis < t.rank:
        raise IndexError(f"Input tensor rank ({t.rank}) must be greater than reduction axis ({axis})")
    if t.size == 0:
        return empty(t.shape, np.int64), empty(t.shape, t.dtype)
    shape = list(t.shape)
    shape[axis] = 1
    idx, val = empty(shape, np.int64), empty(shape, t.dtype)
    check(getattr(_lib.load(), f"am_hip_argreduce_{t.sfx}")(
        RED[op], t.rank, i64_array(t.shape), axis, ctypes.c_void_p(idx.data_ptr()), i64_array(idx.strides),
        ctypes.c_void_p(val.data_ptr()), i64_array(val.strides), ctypes.c_void_p(t.data_ptr()), i64_array(t.strides)))
    return idx, val


def argmax_max(t: HipTensor, axis: int):
    """(indices, maxes) along an axis (src/arraymancer/tensor/aggregate.nim:159-193): the first
    maximum wins; indices are int64, both results keep the axis with extent 1."""
    return _argreduce("max", t, axis)


def argmax(t: HipTensor, axis: int) -> HipTensor:
    """aggregate.nim:195-214."""
    return _argreduce("max", t, axis)[0]


def argmin_min(t: HipTensor, axis: int):
    """(indices, mins) along an axis (aggregate.nim:216-250): the first minimum wins."""
    return _argreduce("min", t, axis)


def argmin(t: HipTensor, axis: int) -> HipTensor:
    """aggregate.nim:252-271."""
    return _argreduce("min", t, axis)[0]


def reduce_all(op, t: HipTensor):
    """reduce_inline (higher_order_foldreduce.nim:22-31): fold of every element, returned to the host."""
    sfx = t.ring_sfx if op in _RING_RED else t.sfx
    out = CTYPE[sfx]()
    check(getattr(_lib.load(), f"am_hip_reduce_all_{sfx}")(
        RED[op], t.rank, i64_array(t.shape), ctypes.c_void_p(t.data_ptr()), i64_array(t.strides), ctypes.byref(out)))
    return _host_scalar(t.dtype, out.value)


def _aggregate(op):
    def f(t: HipTensor, axis: int | None = None):
        return reduce_all(op, t) if axis is None else reduce_axis(op, t, axis)
    f.__name__ = op
    f.__doc__ = f"{op} of all elements (scalar on the host) or along `axis` (src/arraymancer/tensor/aggregate.nim:33-113)."
    return f


# exported by the package as sum / product / min / max (the reference's names); other names here
# so that this module's own use of the builtins stays intact
tsum = _aggregate("sum")
tproduct = _aggregate("product")
tmin = _aggregate("min")
tmax = _aggregate("max")


def mean(t: HipTensor, axis: int | None = None):
    """aggregate.nim:58-86: the sum divided by the element count; integer tensors use `div`."""
    if t.dtype in _UNSIGNED_TWIN:
        raise TypeError("mean divides, which reads the sign of its operands: not defined on unsigned HipTensors")
    if axis is None:
        s = reduce_all("sum", t)
        if t.dtype.kind == "f":
            return t.dtype.type(s / t.dtype.type(t.size))
        q = abs(int(s)) // t.size               # truncation towards zero, like Nim's div
        return t.dtype.type(q if int(s) >= 0 else -q)
    if t.size == 0:
        return empty(t.shape, t.dtype)
    return scalar_op("div", reduce_axis("sum", t, axis), t.dtype.type(t.shape[axis]))


def variance(t: HipTensor, axis: int | None = None):
    """Sample variance, normalised by n - 1 (src/arraymancer/tensor/aggregate.nim:115-146): the mean,
    then the sum of square(y - mean) (one fused map, one fold), divided by n - 1. Floats only."""
    if t.dtype.kind != "f":
        raise TypeError("variance is defined for float tensors")
    if axis is None:
        m = mean(t)
        sq = empty(t.shape, t.dtype)
        _scalar_sqdiff(sq, t, m)
        return t.dtype.type(reduce_all("sum", sq) / t.dtype.type(t.size - 1))
    if t.size == 0:
        return empty(t.shape, t.dtype)
    m = mean(t, axis)
    sq = map2("sqdiff", t, m.broadcast(t.shape))
    return scalar_op("div", reduce_axis("sum", sq, axis), t.dtype.type(t.shape[axis] - 1))


def _scalar_sqdiff(dst: HipTensor, t: HipTensor, m):
    """dst = square(t - m) for a host scalar m: a subtraction pass, then the square in place."""
    _scalar_into("sub", dst, t, m, False)
    _unary_into("square", dst, dst)


def std(t: HipTensor, axis: int | None = None):
    """sqrt of the variance (aggregate.nim:148-158)."""
    v = variance(t, axis)
    if axis is None:
        return t.dtype.type(np.sqrt(v))
    return unary("sqrt", v) if v.size else v


def sqrt(t: HipTensor) -> HipTensor:
    """src/arraymancer/tensor/ufunc.nim:91."""
    return unary("sqrt", t)


def square(t: HipTensor) -> HipTensor:
    """src/arraymancer/tensor/math_functions.nim:218-222."""
    return unary("square", t)


def softmax(t: HipTensor) -> HipTensor:
    """Row softmax of a [batch_size, number_of_classes] matrix
    (src/arraymancer/nn_primitives/nnp_softmax.nim:18-38)."""
    if t.rank != 2:
        raise ValueError("softmax: input must be [batch_size, number_of_classes]")
    if t.dtype.kind != "f":
        raise TypeError("softmax is defined for float tensors")
    out = empty(t.shape, t.dtype)
    check(getattr(_lib.load(), f"am_hip_softmax_rows_{t.sfx}")(
        t.shape[0], t.shape[1], ctypes.c_void_p(out.data_ptr()), *out.strides, ctypes.c_void_p(t.data_ptr()), *t.strides))
    return out


def _check_input_target(input: HipTensor, target: HipTensor, sparse: bool):
    if input.rank != 2 or input.dtype.kind != "f":
        raise ValueError("softmax cross-entropy: input must be a float [batch_size, number_of_classes] matrix")
    if sparse:
        if target.rank != 1 or target.shape[0] != input.shape[0]:
            raise ValueError(f"sparse softmax cross-entropy: {target.shape[0] if target.rank else 0} labels for {input.shape[0]} rows")
        if target.dtype != np.dtype(np.int64):
            raise TypeError("sparse softmax cross-entropy: the labels must be an int64 tensor (the reference's Tensor[int])")
    else:
        _same_dtype(input, target)
        if target.shape != input.shape:     # check_input_target, private/p_nnp_checks.nim
            raise ValueError(f"softmax cross-entropy: input {input.shape} and target {target.shape} must have the same shape")


def softmax_cross_entropy(input: HipTensor, target: HipTensor) -> float:
    """Softmax + cross-entropy loss in one pass, averaged over the batch
    (src/arraymancer/nn_primitives/nnp_softmax_cross_entropy.nim:17-86). `target` holds probabilities [batch, classes]."""
    _check_input_target(input, target, False)
    loss = _lib.CTYPE[input.sfx]()
    check(getattr(_lib.load(), f"am_hip_softmax_cross_entropy_{input.sfx}")(
        input.shape[0], input.shape[1], ctypes.c_void_p(input.data_ptr()), *input.strides,
        ctypes.c_void_p(target.data_ptr()), *target.strides, ctypes.byref(loss)))
    return input.dtype.type(loss.value)


def sparse_softmax_cross_entropy(input: HipTensor, target: HipTensor) -> float:
    """The same loss with one int64 class index per row (nnp_softmax_cross_entropy.nim:88-177)."""
    _check_input_target(input, target, True)
    loss = _lib.CTYPE[input.sfx]()
    check(getattr(_lib.load(), f"am_hip_sparse_softmax_cross_entropy_{input.sfx}")(
        input.shape[0], input.shape[1], ctypes.c_void_p(input.data_ptr()), *input.strides,
        ctypes.c_void_p(target.data_ptr()), target.strides[0], ctypes.byref(loss)))
    return input.dtype.type(loss.value)


def sigmoid_cross_entropy(input: HipTensor, target: HipTensor) -> float:
    """Sigmoid + binary cross-entropy in one pass, averaged over the batch
    (src/arraymancer/nn_primitives/nnp_sigmoid_cross_entropy.nim:23-45)."""
    _check_input_target(input, target, False)
    if input.shape[0] == 0:
        raise ValueError("sigmoid_cross_entropy: empty batch")
    loss = _lib.CTYPE[input.sfx]()
    check(getattr(_lib.load(), f"am_hip_sigmoid_cross_entropy_{input.sfx}")(
        input.shape[0], input.shape[1], ctypes.c_void_p(input.data_ptr()), *input.strides,
        ctypes.c_void_p(target.data_ptr()), *target.strides, ctypes.byref(loss)))
    return input.dtype.type(loss.value)


def sigmoid_cross_entropy_backward(gradient, cached_tensor: HipTensor, target: HipTensor) -> HipTensor:
    """gradient * (sigmoid(cached_tensor) - target) / batch_size (nnp_sigmoid_cross_entropy.nim:47-62)."""
    _check_input_target(cached_tensor, target, False)
    out = empty(cached_tensor.shape, cached_tensor.dtype)
    check(getattr(_lib.load(), f"am_hip_sigmoid_cross_entropy_backward_{cached_tensor.sfx}")(
        cached_tensor.shape[0], cached_tensor.shape[1], _lib.CTYPE[cached_tensor.sfx](_scalar_gradient(gradient, cached_tensor.dtype)),
        ctypes.c_void_p(cached_tensor.data_ptr()), *cached_tensor.strides, ctypes.c_void_p(target.data_ptr()), *target.strides,
        ctypes.c_void_p(out.data_ptr()), *out.strides))
    return out


def _scalar_gradient(gradient, dtype):
    """The reference takes the upstream gradient as a scalar or as a one-element tensor (its first element is used)."""
    if isinstance(gradient, HipTensor):
        return dtype.type(gradient.toCpu().reshape(-1)[0])
    return dtype.type(gradient)


def softmax_cross_entropy_backward(gradient, cached_tensor: HipTensor, target: HipTensor) -> HipTensor:
    """gradient * (softmax(cached_tensor) - target) / batch_size in one launch
    (nnp_softmax_cross_entropy.nim:186-214)."""
    _check_input_target(cached_tensor, target, False)
    out = empty(cached_tensor.shape, cached_tensor.dtype)
    check(getattr(_lib.load(), f"am_hip_softmax_cross_entropy_backward_{cached_tensor.sfx}")(
        cached_tensor.shape[0], cached_tensor.shape[1], _lib.CTYPE[cached_tensor.sfx](_scalar_gradient(gradient, cached_tensor.dtype)),
        ctypes.c_void_p(cached_tensor.data_ptr()), *cached_tensor.strides, ctypes.c_void_p(target.data_ptr()), *target.strides,
        ctypes.c_void_p(out.data_ptr()), *out.strides))
    return out


def sparse_softmax_cross_entropy_backward(gradient, cached_tensor: HipTensor, target: HipTensor) -> HipTensor:
    """gradient * (softmax(cached_tensor) - onehot(target)) / batch_size in one launch
    (nnp_softmax_cross_entropy.nim:217-256)."""
    _check_input_target(cached_tensor, target, True)
    out = empty(cached_tensor.shape, cached_tensor.dtype)
    check(getattr(_lib.load(), f"am_hip_sparse_softmax_cross_entropy_backward_{cached_tensor.sfx}")(
        cached_tensor.shape[0], cached_tensor.shape[1], _lib.CTYPE[cached_tensor.sfx](_scalar_gradient(gradient, cached_tensor.dtype)),
        ctypes.c_void_p(cached_tensor.data_ptr()), *cached_tensor.strides, ctypes.c_void_p(target.data_ptr()), target.strides[0],
        ctypes.c_void_p(out.data_ptr()), *out.strides))
    return out


def maxpool2d(x: HipTensor, kernel, padding=(0, 0), stride=(1, 1)):
    """(max_indices, maxpooled) of a C-contiguous [N, C, H, W] tensor
    (src/arraymancer/nn_primitives/nnp_maxpooling.nim:19-66; the reference asserts contiguity too).
    max_indices is a device int64 vector of flat input indices."""
    if x.rank != 4 or not x.is_C_contiguous():
        raise ValueError("maxpool2d: input must be a C-contiguous [N, C, H, W] tensor")
    N, C, H, W = x.shape
    (kh, kw), (ph, pw), (sh, sw) = kernel, padding, stride
    ho, wo = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
    out = empty((N, C, ho, wo), x.dtype)
    idx = empty((N * C * ho * wo,), np.int64)
    check(getattr(_lib.load(), f"am_hip_maxpool2d_{x.sfx}")(
        N, C, H, W, kh, kw, ph, pw, sh, sw, ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(out.data_ptr()),
        ctypes.c_void_p(idx.data_ptr())))
    idx.pool_geometry = ((kh, kw), (ph, pw), (sh, sw))   # what maxpool2d_backward needs besides the indices
    return idx, out


def maxpool2d_backward(cached_input_shape, cached_max_indices: HipTensor, gradOutput: HipTensor, kernel=None,
                       padding=None, stride=None) -> HipTensor:
    """gradInput = zeros(cached_input_shape) with gradInput[max_indices[i]] = gradOutput[i]
    (src/arraymancer/nn_primitives/nnp_maxpooling.nim:68-83). The device runs the scatter as a gather
    over the pooling windows and therefore needs kernel, padding and stride: they are taken from
    the indices returned by maxpool2d of this module, or passed explicitly."""
    geom = getattr(cached_max_indices, "pool_geometry", None)
    if kernel is not None:
        geom = (tuple(kernel), tuple(padding or (0, 0)), tuple(stride or (1, 1)))
    if geom is None:
        raise ValueError("maxpool2d_backward: pass kernel, padding and stride (the indices do not come from maxpool2d)")
    shape = tuple(int(s) for s in cached_input_shape)
    if len(shape) != 4:
        raise ValueError("maxpool2d_backward: cached_input_shape must be [N, C, H, W]")
    (kh, kw), (ph, pw), (sh, sw) = geom
    N, C, H, W = shape
    ho, wo = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
    if gradOutput.size != cached_max_indices.size or gradOutput.size != N * C * ho * wo:
        raise ValueError("maxpool2d_backward: gradOutput, the indices and the pooling geometry do not match")
    if cached_max_indices.dtype != np.int64 or not cached_max_indices.is_C_contiguous() or not gradOutput.is_C_contiguous():
        raise ValueError("maxpool2d_backward: indices must be a contiguous int64 tensor, gradOutput contiguous")
    out = empty(shape, gradOutput.dtype)
    check(getattr(_lib.load(), f"am_hip_maxpool2d_backward_{gradOutput.sfx}")(
        N, C, H, W, kh, kw, ph, pw, sh, sw, ctypes.c_void_p(cached_max_indices.data_ptr()),
        ctypes.c_void_p(gradOutput.data_ptr()), ctypes.c_void_p(out.data_ptr())))
    return out

