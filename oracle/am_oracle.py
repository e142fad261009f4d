"""TEST INFRASTRUCTURE — ctypes front end of the CPU oracle (oracle/libam_oracle.so) plus
closed-form NumPy checks that pin it.

Only tests, ``__graft_entry__.smoke()`` and the CPU-baseline leg of ``bench.py`` may import this
module. Nothing under ``arraymancer_amd/`` does: the product path runs on the HIP library only.

The C library restates the reference's algorithms (see the headers of laser_gemm.c and
strided_map.c for the file:line map). The functions named ``closed_*`` below do NOT restate the
reference: they compute what the mathematics fixes (modular integer products, higher-precision
float products, NumPy broadcasting) and are what the restatement is checked against.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from fractions import Fraction

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libam_oracle.so")

_SFX = {np.dtype(np.float32): "f32", np.dtype(np.float64): "f64",
        np.dtype(np.int32): "i32", np.dtype(np.int64): "i64"}
_CT = {"f32": ctypes.c_float, "f64": ctypes.c_double, "i32": ctypes.c_int32, "i64": ctypes.c_int64}

# op codes of include/am_hip.h
OP = dict(add=0, sub=1, mul=2, div=3, mod=4, add_relu=5, add_sigmoid=6, add_tanh=7,
          relu_bwd=8, max=9, min=10, sigmoid_bwd=11, tanh_bwd=12, sqdiff=13, pow=14, floormod=15, copysign=16)
CMP = {"==": 0, "!=": 1, "<": 2, "<=": 3, ">": 4, ">=": 5, "mod_is_zero": 6}
PRED = dict(isnan=0, isnotnan=1, classify=2)
OP3 = dict(muladd=0, gru_candidate=1, gru_blend=2, addmul=3, clamp=4)
UOP = dict(copy=0, neg=1, relu=2, sigmoid=3, tanh=4, exp=5, abs=6, sqrt=7, square=8,
           ln=9, log10=10, log2=11, sin=12, cos=13, tan=14, sinh=15, cosh=16, arcsin=17,
           arccos=18, arctan=19, arcsinh=20, arccosh=21, arctanh=22, cbrt=23, erf=24, erfc=25, gamma=26,
           lgamma=27, floor=28, ceil=29, trunc=30, round=31, reciprocal=32, degtorad=33, radtodeg=34, fac=35)


def build(force: bool = False) -> str:
    """Compile the oracle with its Makefile (gcc). Returns the library path."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s", "libam_oracle.so"],
                       check=True, capture_output=True)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        i64, p, ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
        for sfx, ct in _CT.items():
            f = getattr(L, f"am_oracle_gemm_strided_{sfx}")
            f.restype = ci
            f.argtypes = [i64, i64, i64, ct, p, i64, i64, p, i64, i64, ct, p, i64, i64]
            f = getattr(L, f"am_oracle_map2_{sfx}")
            f.restype = ci
            f.argtypes = [ci, ci, p, p, p, p, p, p, p]
            f = getattr(L, f"am_oracle_map3_{sfx}")
            f.restype = ci
            f.argtypes = [ci, ci, p, p, p, p, p, p, p, p, p]
            f = getattr(L, f"am_oracle_scalar_{sfx}")
            f.restype = ci
            f.argtypes = [ci, ci, ci, p, p, p, p, p, ct]
            f = getattr(L, f"am_oracle_unary_{sfx}")
            f.restype = ci
            f.argtypes = [ci, ci, p, p, p, p, p]
            f = getattr(L, f"am_oracle_compare_{sfx}")
            f.restype = ci
            f.argtypes = [ci, ci, p, p, p, p, p, p, p]
            f = getattr(L, f"am_oracle_sgn_{sfx}")
            f.restype = ci
            f.argtypes = [ci, p, p, p, p, p]
            f = getattr(L, f"am_oracle_reduce_axis_{sfx}")
            f.restype = ci
            f.argtypes = [ci, ci, p, ci, p, p, p, p]
            f = getattr(L, f"am_oracle_argreduce_{sfx}")
            f.restype = ci
            f.argtypes = [ci, ci, p, ci, p, p, p, p, p, p]
            f = getattr(L, f"am_oracle_reduce_all_{sfx}")
            f.restype = ci
            f.argtypes = [ci, ci, p, p, p, p]
            f = getattr(L, f"am_oracle_maxpool2d_backward_{sfx}")
            f.restype = ci
            f.argtypes = [i64, i64, p, p, p]
            f = getattr(L, f"am_oracle_maxpool2d_{sfx}")
            f.restype = ci
            f.argtypes = [i64, ci, ci, ci, ci, ci, ci, ci, ci, ci, p, p, p, ct]
        for sfx in ("f32", "f64"):
            f = getattr(L, f"am_oracle_predicate_{sfx}")
            f.restype = ci
            f.argtypes = [ci, ci, p, p, p, p, p]
            f = getattr(L, f"am_oracle_softmax_rows_{sfx}")
            f.restype = ci
            f.argtypes = [i64, i64, p, i64, i64, p, i64, i64]
        L.am_oracle_num_threads.restype = ci
        L.am_oracle_set_num_threads.argtypes = [ci]
        _lib = L
    return _lib


def num_threads() -> int:
    return lib().am_oracle_num_threads()


def set_num_threads(n: int) -> None:
    lib().am_oracle_set_num_threads(int(n))


def _sfx(arr: np.ndarray) -> str:
    try:
        return _SFX[arr.dtype]
    except KeyError:
        raise TypeError(f"oracle supports float32/float64/int32/int64, not {arr.dtype}")


def _estrides(arr: np.ndarray):
    it = arr.dtype.itemsize
    assert all(s % it == 0 for s in arr.strides)
    return [s // it for s in arr.strides]


def _i64arr(vals):
    return (ctypes.c_int64 * max(1, len(vals)))(*vals)


# ----------------------------------------------------------------------------- restatement
def gemm_strided(alpha, A: np.ndarray, B: np.ndarray, beta, C: np.ndarray) -> np.ndarray:
    """C <- alpha*A*B + beta*C in place through laser's blocked algorithm. A, B, C are rank-2
    NumPy arrays or views (any strides, incl. negative and zero for A/B); C is written through
    its own strides. Returns C."""
    assert A.ndim == B.ndim == C.ndim == 2 and A.dtype == B.dtype == C.dtype
    M, K = A.shape
    K2, N = B.shape
    assert K == K2 and C.shape == (M, N)
    sfx = _sfx(A)
    ct = _CT[sfx]
    (rsa, csa), (rsb, csb), (rsc, csc) = _estrides(A), _estrides(B), _estrides(C)
    rc = getattr(lib(), f"am_oracle_gemm_strided_{sfx}")(
        M, N, K, ct(alpha), A.ctypes.data, rsa, csa, B.ctypes.data, rsb, csb,
        ct(beta), C.ctypes.data, rsc, csc)
    if rc != 0:
        raise MemoryError("oracle gemm_strided: packing buffers")
    return C


def matmul(A: np.ndarray, B: np.ndarray) -> np.ndarray:
    """`*` of the Tensor API: fresh row-major C, gemm(1, A, B, 0, C)
    (src/arraymancer/tensor/operators_blas_l2l3.nim:88-100)."""
    C = np.empty((A.shape[0], B.shape[1]), dtype=A.dtype)
    C.fill(np.nan if C.dtype.kind == "f" else -77)   # beta == 0 must overwrite whatever is there
    return gemm_strided(1, A, B, 0, C)


def broadcast2(a: np.ndarray, b: np.ndarray):
    """broadcast2Impl (src/arraymancer/tensor/private/p_shapeshifting.nim:96-134): equal ranks,
    size-1 axes get stride 0; anything else raises ValueError."""
    if a.ndim != b.ndim:
        raise ValueError("broadcast2: ranks differ")
    shape = []
    for sa, sb in zip(a.shape, b.shape):
        if sa == sb or sb == 1:
            shape.append(sa)
        elif sa == 1:
            shape.append(sb)
        else:
            raise ValueError(f"Broadcasting error: non-singleton dimensions must be the same in both tensors. "
                             f"Tensors' shapes were: {a.shape} and {b.shape}")
    return _bc(a, shape), _bc(b, shape)


def _bc(t: np.ndarray, shape):
    strides = [0 if (ts == 1 and s != 1) else st for ts, s, st in zip(t.shape, shape, t.strides)]
    return np.lib.stride_tricks.as_strided(t, shape=tuple(shape), strides=tuple(strides), writeable=False)


def broadcast(t: np.ndarray, shape):
    """broadcastImpl (p_shapeshifting.nim:76-94)."""
    if t.ndim != len(shape):
        raise ValueError("broadcast: ranks differ")
    for ts, s in zip(t.shape, shape):
        if ts != 1 and ts != s:
            raise ValueError(f"The broadcasted size of the tensor {list(shape)}, must match existing size "
                             f"{list(t.shape)} for non-singleton dimension")
    return _bc(t, shape)


def map2(op, a: np.ndarray, b: np.ndarray, out: np.ndarray | None = None) -> np.ndarray:
    """out[i] = op(a[i], b[i]) over equal shapes, each operand walked in C order through its own
    strides. out=None allocates the fresh contiguous result of map2_inline; out=a is apply2_inline."""
    op = OP[op] if isinstance(op, str) else op
    assert a.shape == b.shape and a.dtype == b.dtype
    if out is None:
        out = np.empty(a.shape, dtype=a.dtype)
    assert out.shape == a.shape and out.dtype == a.dtype
    sfx = _sfx(a)
    rc = getattr(lib(), f"am_oracle_map2_{sfx}")(
        op, a.ndim, _i64arr(a.shape), out.ctypes.data, _i64arr(_estrides(out)),
        a.ctypes.data, _i64arr(_estrides(a)), b.ctypes.data, _i64arr(_estrides(b)))
    if rc != 0:
        raise ValueError(f"oracle map2: op {op} not defined for {a.dtype} (rc={rc})")
    return out


def compare(cmp, a: np.ndarray, b) -> np.ndarray:
    """Bool tensor of a[i] cmp b[i] (equal shapes, or b a scalar seen through zero strides): the broadcast
    comparison family and `x mod y == 0`."""
    if not isinstance(b, np.ndarray):
        b = np.broadcast_to(np.asarray(b, dtype=a.dtype), a.shape)
    assert a.shape == b.shape and a.dtype == b.dtype
    out = np.empty(a.shape, dtype=np.uint8)
    rc = getattr(lib(), f"am_oracle_compare_{_sfx(a)}")(
        CMP[cmp], a.ndim, _i64arr(a.shape), out.ctypes.data, _i64arr(_estrides(out)),
        a.ctypes.data, _i64arr(_estrides(a)), b.ctypes.data, _i64arr(_estrides(b)))
    if rc != 0:
        raise ValueError(f"oracle compare: rc={rc}")
    return out.view(np.bool_)


def predicate(pred, a: np.ndarray) -> np.ndarray:
    """isnan / isnotnan (bool) or classify (uint8 ordinals of Nim's FloatClass) of a float tensor."""
    out = np.empty(a.shape, dtype=np.uint8)
    rc = getattr(lib(), f"am_oracle_predicate_{_sfx(a)}")(
        PRED[pred], a.ndim, _i64arr(a.shape), out.ctypes.data, _i64arr(_estrides(out)),
        a.ctypes.data, _i64arr(_estrides(a)))
    if rc != 0:
        raise ValueError(f"oracle predicate: rc={rc}")
    return out if pred == "classify" else out.view(np.bool_)


def sgn(a: np.ndarray) -> np.ndarray:
    out = np.empty(a.shape, dtype=np.int64)
    rc = getattr(lib(), f"am_oracle_sgn_{_sfx(a)}")(
        a.ndim, _i64arr(a.shape), out.ctypes.data, _i64arr(_estrides(out)), a.ctypes.data, _i64arr(_estrides(a)))
    if rc != 0:
        raise ValueError(f"oracle sgn: rc={rc}")
    return out


def map3(op, a: np.ndarray, b: np.ndarray, c: np.ndarray, out: np.ndarray | None = None) -> np.ndarray:
    """out[i] = op(a[i], b[i], c[i]); out=a is apply3_inline."""
    op = OP3[op] if isinstance(op, str) else op
    assert a.shape == b.shape == c.shape and a.dtype == b.dtype == c.dtype
    if out is None:
        out = np.empty(a.shape, dtype=a.dtype)
    sfx = _sfx(a)
    rc = getattr(lib(), f"am_oracle_map3_{sfx}")(
        op, a.ndim, _i64arr(a.shape), out.ctypes.data, _i64arr(_estrides(out)),
        a.ctypes.data, _i64arr(_estrides(a)), b.ctypes.data, _i64arr(_estrides(b)),
        c.ctypes.data, _i64arr(_estrides(c)))
    if rc != 0:
        raise ValueError(f"oracle map3: op {op} not defined for {a.dtype} (rc={rc})")
    return out


def scalar_op(op, a: np.ndarray, scalar, scalar_on_left=False, out: np.ndarray | None = None) -> np.ndarray:
    op = OP[op] if isinstance(op, str) else op
    if out is None:
        out = np.empty(a.shape, dtype=a.dtype)
    sfx = _sfx(a)
    rc = getattr(lib(), f"am_oracle_scalar_{sfx}")(
        op, int(bool(scalar_on_left)), a.ndim, _i64arr(a.shape), out.ctypes.data,
        _i64arr(_estrides(out)), a.ctypes.data, _i64arr(_estrides(a)), _CT[sfx](scalar))
    if rc != 0:
        raise ValueError(f"oracle scalar_op: op {op} not defined for {a.dtype} (rc={rc})")
    return out


def unary(op, a: np.ndarray, out: np.ndarray | None = None) -> np.ndarray:
    op = UOP[op] if isinstance(op, str) else op
    if out is None:
        out = np.empty(a.shape, dtype=a.dtype)
    sfx = _sfx(a)
    rc = getattr(lib(), f"am_oracle_unary_{sfx}")(
        op, a.ndim, _i64arr(a.shape), out.ctypes.data, _i64arr(_estrides(out)),
        a.ctypes.data, _i64arr(_estrides(a)))
    if rc != 0:
        raise ValueError(f"oracle unary: op {op} not defined for {a.dtype} (rc={rc})")
    return out


def im2col(img: np.ndarray, kernel_size, padding=(0, 0), stride=(1, 1)) -> np.ndarray:
    """im2col of ONE image [C, H, W] -> [C*kH*kW, H_out*W_out], loop for loop as the reference
    (src/arraymancer/nn_primitives/fallback/conv.nim:18-54)."""
    C, H, W = img.shape
    (kh, kw), (ph, pw), (sh, sw) = kernel_size, padding, stride
    hc, wc = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
    out = np.zeros((C * kh * kw, hc * wc), dtype=img.dtype)
    flat = img.reshape(-1)
    for c in range(C * kh * kw):
        w_off, h_off, c_off = c % kw - pw, (c // kw) % kh - ph, (c // kw) // kh
        for h in range(hc):
            row = h_off + h * sh
            for w in range(wc):
                col = w_off + w * sw
                if 0 <= row < H and 0 <= col < W:
                    out[c, h * wc + w] = flat[c_off * H * W + row * W + col]
    return out


def conv2d(x: np.ndarray, kernel: np.ndarray, bias: np.ndarray | None, padding=(0, 0), stride=(1, 1)) -> np.ndarray:
    """im2colgemm_conv2d (fallback/conv.nim:81-106): per image im2col, gemm(1, kernel_col, input_col,
    0, out_view) through the restated laser GEMM, then result +.= bias.unsqueeze(0)."""
    N, C, H, W = x.shape
    co, _, kh, kw = kernel.shape
    ho, wo = (H + 2 * padding[0] - kh) // stride[0] + 1, (W + 2 * padding[1] - kw) // stride[1] + 1
    kcol = np.ascontiguousarray(kernel.reshape(co, C * kh * kw))
    out = np.empty((N, co, ho, wo), dtype=x.dtype)
    for n in range(N):
        col = im2col(np.ascontiguousarray(x[n]), (kh, kw), padding, stride)
        gemm_strided(1, kcol, col, 0, out[n].reshape(co, ho * wo))
    if bias is not None:
        b = broadcast(bias.reshape(1, co, 1, 1), out.shape)
        map2("add", out, b, out=out)
    return out


def col2im(col: np.ndarray, channels: int, height: int, width: int, kernel_size, padding=(0, 0), stride=(1, 1)) -> np.ndarray:
    """col2im of ONE column matrix [C*kH*kW, H_out*W_out] -> [C, H, W], loop for loop as the reference
    (src/arraymancer/nn_primitives/fallback/conv.nim:55-79): pixels that several columns cover are summed, in
    the order of the rows of the column matrix."""
    (kh, kw), (ph, pw), (sh, sw) = kernel_size, padding, stride
    hc, wc = (height + 2 * ph - kh) // sh + 1, (width + 2 * pw - kw) // sw + 1
    out = np.zeros((channels, height, width), dtype=col.dtype)
    with np.errstate(over="ignore"):
        for c in range(channels * kh * kw):
            w_off, h_off, c_off = c % kw - pw, (c // kw) % kh - ph, (c // kw) // kh
            for h in range(hc):
                row = h_off + h * sh
                if not 0 <= row < height:
                    continue
                for w in range(wc):
                    cc = w_off + w * sw
                    if 0 <= cc < width:
                        out[c_off, row, cc] += col[c, h * wc + w]
    return out


def conv2d_backward(x: np.ndarray, kernel: np.ndarray, bias: np.ndarray | None, padding, stride, grad_output: np.ndarray):
    """conv2d_backward (src/arraymancer/nn_primitives/nnp_convolution.nim:65-107) over
    im2colgemm_conv2d_gradient (fallback/conv.nim:107-145): per image grad_input_col = kernel_col^T * grad_output_col,
    grad_input[n] = col2im(grad_input_col), grad_weight += grad_output_col * input_col^T, all through the restated laser
    GEMM; grad_bias = grad_output.sum(3).sum(2).sum(0). Returns (grad_input, grad_weight, grad_bias or None)."""
    N, C, H, W = x.shape
    co, _, kh, kw = kernel.shape
    ho, wo = (H + 2 * padding[0] - kh) // stride[0] + 1, (W + 2 * padding[1] - kw) // stride[1] + 1
    assert grad_output.shape == (N, co, ho, wo)
    kcol = np.ascontiguousarray(kernel.reshape(co, C * kh * kw))
    grad_input = np.zeros_like(x)
    grad_weight = np.zeros((co, C * kh * kw), dtype=x.dtype)
    for n in range(N):
        gcol = np.ascontiguousarray(grad_output[n].reshape(co, ho * wo))
        gin_col = np.empty((C * kh * kw, ho * wo), dtype=x.dtype)
        gemm_strided(1, kcol.T, gcol, 0, gin_col)
        grad_input[n] = col2im(gin_col, C, H, W, (kh, kw), padding, stride)
        col = im2col(np.ascontiguousarray(x[n]), (kh, kw), padding, stride)
        part = np.empty_like(grad_weight)
        gemm_strided(1, gcol, col.T, 0, part)
        map2("add", grad_weight, part, out=grad_weight)
    grad_bias = None
    if bias is not None:
        g = grad_output
        for ax in (3, 2, 0):
            g = reduce_axis("sum", np.ascontiguousarray(g), ax)
        grad_bias = g.reshape(bias.shape)
    return grad_input, grad_weight.reshape(kernel.shape), grad_bias


# ----------------------------------------------------------------------------- closed forms
RED = {"sum": 0, "product": 1, "min": 2, "max": 3}


def reduce_axis(op, a: np.ndarray, axis: int) -> np.ndarray:
    """reduce_axis_inline (higher_order_foldreduce.nim:46-61): fold along `axis` starting from the
    first slice; the result keeps the axis with extent 1. Any strides."""
    sfx = _sfx(a)
    if not 0 <= axis < a.ndim:
        raise IndexError(f"axis {axis} outside rank {a.ndim}")
    out_shape = list(a.shape)
    out_shape[axis] = 1
    out = np.empty(out_shape, dtype=a.dtype)
    if a.size == 0:
        return np.empty(a.shape, dtype=a.dtype)
    rc = getattr(lib(), f"am_oracle_reduce_axis_{sfx}")(
        RED[op], a.ndim, _i64arr(a.shape), axis, out.ctypes.data, _i64arr(_estrides(out)), a.ctypes.data, _i64arr(_estrides(a)))
    if rc != 0:
        raise ValueError(f"oracle reduce_axis failed ({rc})")
    return out


def argreduce(op, a: np.ndarray, axis: int):
    """argmax_max (op "max") / argmin_min (op "min") of tensor/aggregate.nim:159-193, 216-250:
    (indices as int64, values), both with extent 1 along `axis`."""
    sfx = _sfx(a)
    if not 0 <= axis < a.ndim:
        raise IndexError(f"axis {axis} outside rank {a.ndim}")
    out_shape = list(a.shape)
    out_shape[axis] = 1
    if a.size == 0:
        return np.empty(a.shape, dtype=np.int64), np.empty(a.shape, dtype=a.dtype)
    idx, val = np.empty(out_shape, dtype=np.int64), np.empty(out_shape, dtype=a.dtype)
    rc = getattr(lib(), f"am_oracle_argreduce_{sfx}")(
        RED[op], a.ndim, _i64arr(a.shape), axis, idx.ctypes.data, _i64arr(_estrides(idx)), val.ctypes.data,
        _i64arr(_estrides(val)), a.ctypes.data, _i64arr(_estrides(a)))
    if rc != 0:
        raise ValueError(f"oracle argreduce failed ({rc})")
    return idx, val


def reduce_all(op, a: np.ndarray):
    """reduce_inline (higher_order_foldreduce.nim:22-31): C-order fold from the first element."""
    sfx = _sfx(a)
    if a.size == 0:
        raise ValueError("reduction of an empty tensor")
    res = np.empty(1, dtype=a.dtype)
    rc = getattr(lib(), f"am_oracle_reduce_all_{sfx}")(RED[op], a.ndim, _i64arr(a.shape), a.ctypes.data, _i64arr(_estrides(a)), res.ctypes.data)
    if rc != 0:
        raise ValueError(f"oracle reduce_all failed ({rc})")
    return res[0]


def mean(a: np.ndarray, axis: int | None = None):
    """aggregate.nim:58-80: sum divided by the element count; integers use `div` (truncation)."""
    if axis is None:
        s, n = reduce_all("sum", a), a.size
    else:
        s, n = reduce_axis("sum", a, axis), a.shape[axis]
    if a.dtype.kind == "f":
        return (s / a.dtype.type(n)).astype(a.dtype) if isinstance(s, np.ndarray) else a.dtype.type(s / a.dtype.type(n))
    q = _trunc_div(np.asarray(s), np.asarray(n, dtype=a.dtype))
    return q if axis is not None else q.dtype.type(q)


def variance(a: np.ndarray, axis: int | None = None):
    """aggregate.nim:115-146: mean, then the serial fold of square(y - mean) in the tensor's own
    precision, divided by n - 1."""
    m = mean(a, axis)
    d = a - m                      # m broadcasts: it keeps the reduced axis with extent 1
    sq = (d * d).astype(a.dtype)
    if axis is None:
        return a.dtype.type(reduce_all("sum", sq) / a.dtype.type(a.size - 1))
    return (reduce_axis("sum", sq, axis) / a.dtype.type(a.shape[axis] - 1)).astype(a.dtype)


def std(a: np.ndarray, axis: int | None = None):
    """aggregate.nim:148-158."""
    v = variance(a, axis)
    return np.sqrt(v).astype(a.dtype) if axis is not None else a.dtype.type(np.sqrt(v))


def softmax(x: np.ndarray) -> np.ndarray:
    """nnp_softmax.nim:18-38 on a [batch, classes] matrix (streaming max / sum of exponentials per
    row, then exp(x - max) / sumexp)."""
    sfx = _sfx(x)
    assert x.ndim == 2 and sfx in ("f32", "f64")
    out = np.empty(x.shape, dtype=x.dtype)
    xs, os_ = _estrides(x), _estrides(out)
    getattr(lib(), f"am_oracle_softmax_rows_{sfx}")(x.shape[0], x.shape[1], out.ctypes.data, os_[0], os_[1], x.ctypes.data, xs[0], xs[1])
    return out


def streaming_max_sumexp(x: np.ndarray):
    """Row by row the one-pass recurrence of streaming_max_sumexp (src/arraymancer/nn_primitives/private/
    p_logsumexp.nim:20-31), in the element type: the running maximum and the sum of exp(x - maximum), rescaled whenever
    the maximum moves. All rows advance together, each through its own elements in order. Returns (max, sumexp)."""
    dt = x.dtype.type
    mx = np.full(x.shape[0], -np.inf, dtype=x.dtype)
    se = np.zeros(x.shape[0], dtype=x.dtype)
    with np.errstate(over="ignore", invalid="ignore"):
        for j in range(x.shape[1]):
            val = x[:, j]
            le = val <= mx
            se = np.where(le, se + np.exp(val - mx), se * np.exp(mx - val) + dt(1)).astype(x.dtype)
            mx = np.where(le, mx, val)
    return mx, se


def softmax_cross_entropy(x: np.ndarray, target: np.ndarray):
    """softmax_cross_entropy (src/arraymancer/nn_primitives/nnp_softmax_cross_entropy.nim:17-86): per row
    ln(sumexp) + max - dot(row, target row), summed over the rows in order, divided by the batch size."""
    dt = x.dtype.type
    if x.shape[0] == 0:
        return dt(0)
    mx, se = streaming_max_sumexp(x)
    dot = np.zeros(x.shape[0], dtype=x.dtype)
    for j in range(x.shape[1]):
        dot = (dot + x[:, j] * target[:, j]).astype(x.dtype)
    local = (np.log(se) + mx - dot).astype(x.dtype)
    total = dt(0)
    for v in local:
        total = dt(total + v)
    return dt(total / dt(x.shape[0]))


def sparse_softmax_cross_entropy(x: np.ndarray, labels: np.ndarray):
    """sparse_softmax_cross_entropy (nnp_softmax_cross_entropy.nim:88-177): per row ln(sumexp) + max - row[label]."""
    dt = x.dtype.type
    if x.shape[0] == 0:
        return dt(0)
    mx, se = streaming_max_sumexp(x)
    local = ((np.log(se) + mx).astype(x.dtype) - x[np.arange(x.shape[0]), labels.astype(np.int64)]).astype(x.dtype)
    total = dt(0)
    for v in local:
        total = dt(total + v)
    return dt(total / dt(x.shape[0]))


def softmax_cross_entropy_backward(gradient, x: np.ndarray, target: np.ndarray) -> np.ndarray:
    """softmax_cross_entropy_backward (nnp_softmax_cross_entropy.nim:186-214):
    grad * (exp(x - max) / sumexp - target) / batch_size, every step rounded in the element type."""
    dt = x.dtype.type
    mx, se = streaming_max_sumexp(x)
    sm = (np.exp(x - mx[:, None]) / se[:, None]).astype(x.dtype)
    return ((dt(gradient) * (sm - target)).astype(x.dtype) / dt(x.shape[0])).astype(x.dtype)


def sparse_softmax_cross_entropy_backward(gradient, x: np.ndarray, labels: np.ndarray) -> np.ndarray:
    """sparse_softmax_cross_entropy_backward (nnp_softmax_cross_entropy.nim:217-256): the result starts as -1 at each
    row's label and 0 elsewhere, then grad * (softmax + that) / batch_size."""
    dt = x.dtype.type
    mx, se = streaming_max_sumexp(x)
    sm = (np.exp(x - mx[:, None]) / se[:, None]).astype(x.dtype)
    start = np.zeros_like(x)
    start[np.arange(x.shape[0]), labels.astype(np.int64)] = dt(-1)
    return ((dt(gradient) * (sm + start)).astype(x.dtype) / dt(x.shape[0])).astype(x.dtype)


def sigmoid_cross_entropy(x: np.ndarray, target: np.ndarray):
    """sigmoid_cross_entropy (src/arraymancer/nn_primitives/nnp_sigmoid_cross_entropy.nim:23-45): the map2 body
    -y * x + max(x, 0) + ln1p(exp(-|x|)) in the element type, summed in C order, divided by the batch size."""
    dt = x.dtype.type
    body = (-target * x + np.maximum(x, dt(0)) + np.log1p(np.exp(-np.abs(x)))).astype(x.dtype)
    total = dt(0)
    for v in body.reshape(-1):
        total = dt(total + v)
    return dt(total / dt(x.shape[0]))


def sigmoid_cross_entropy_backward(gradient, x: np.ndarray, target: np.ndarray) -> np.ndarray:
    """sigmoid_cross_entropy_backward (nnp_sigmoid_cross_entropy.nim:47-62): grad * (sigmoid(x) - y) / batch_size with
    sigmoid(x) = 1 / (1 + exp(-x)) (nn_primitives/private/p_activation.nim:17-18)."""
    dt = x.dtype.type
    sg = (dt(1) / (dt(1) + np.exp(-x))).astype(x.dtype)
    return ((dt(gradient) * (sg - target)).astype(x.dtype) / dt(x.shape[0])).astype(x.dtype)


def maxpool2d(x: np.ndarray, kernel, padding=(0, 0), stride=(1, 1)):
    """nnp_maxpooling.nim:19-66: (max_indices [N*C*outH*outW] int64, maxpooled [N, C, outH, outW])."""
    sfx = _sfx(x)
    x = np.ascontiguousarray(x)
    N, C, H, W = x.shape
    outH = (H + 2 * padding[0] - kernel[0]) // stride[0] + 1
    outW = (W + 2 * padding[1] - kernel[1]) // stride[1] + 1
    out = np.empty((N, C, outH, outW), dtype=x.dtype)
    idx = np.empty(N * C * outH * outW, dtype=np.int64)
    lowest = -np.inf if x.dtype.kind == "f" else np.iinfo(x.dtype).min   # low(T)
    getattr(lib(), f"am_oracle_maxpool2d_{sfx}")(N, C, H, W, kernel[0], kernel[1], padding[0], padding[1], stride[0], stride[1],
                                                 x.ctypes.data, out.ctypes.data, idx.ctypes.data, _CT[sfx](lowest))
    return idx, out


def maxpool2d_backward(cached_input_shape, cached_max_indices: np.ndarray, grad_output: np.ndarray) -> np.ndarray:
    """nnp_maxpooling.nim:68-83, serial: zeros(cached_input_shape), then result[idx[i]] = gradOutput[i]
    for i in order."""
    sfx = _sfx(grad_output)
    go = np.ascontiguousarray(grad_output).reshape(-1)
    idx = np.ascontiguousarray(cached_max_indices, dtype=np.int64).reshape(-1)
    assert go.size == idx.size
    out = np.empty(tuple(cached_input_shape), dtype=grad_output.dtype)
    getattr(lib(), f"am_oracle_maxpool2d_backward_{sfx}")(out.size, go.size, idx.ctypes.data, go.ctypes.data, out.ctypes.data)
    return out


def closed_gemm_int(alpha, A, B, beta, C):
    """Exact integer result of alpha*A*B + beta*C reduced modulo 2^w (w = bit width of the dtype).
    Ring arithmetic is order independent, so this fixes every bit of the result. Uses Python
    integers (object arrays): keep the sizes small, or use closed_gemm_int_fast."""
    w = A.dtype.itemsize * 8
    Ao, Bo, Co = A.astype(object), B.astype(object), C.astype(object)
    R = int(alpha) * Ao.dot(Bo) + int(beta) * Co if A.shape[1] > 0 else Co
    return _wrap_obj(R, w).astype(A.dtype)


def _wrap_obj(R, w):
    mod, half = 1 << w, 1 << (w - 1)
    f = np.vectorize(lambda v: ((int(v) + half) % mod) - half, otypes=[object])
    return f(R) if R.size else R


def closed_gemm_int_fast(alpha, A, B, beta, C):
    """Same value as closed_gemm_int through NumPy uint64 arithmetic (wraps modulo 2^64, and
    2^32 divides 2^64, so reducing afterwards is exact for int32 too)."""
    w = A.dtype.itemsize * 8
    Au, Bu, Cu = (x.astype(np.int64).view(np.uint64) for x in (A, B, C))
    with np.errstate(over="ignore"):
        R = np.uint64(int(alpha) % (1 << 64)) * (Au @ Bu) + np.uint64(int(beta) % (1 << 64)) * Cu
    if w == 32:
        return (R & np.uint64(0xFFFFFFFF)).astype(np.uint32).view(np.int32)
    return R.view(np.int64)


def closed_gemm_float(alpha, A, B, beta, C, dtype=np.longdouble):
    """alpha*A*B + beta*C evaluated in a wider type (float64 for float32 inputs is enough;
    long double for float64 inputs). beta == 0 ignores C, as the reference does."""
    Aw, Bw = A.astype(dtype), B.astype(dtype)
    R = dtype(alpha) * (Aw @ Bw)
    if beta != 0:
        R = R + dtype(beta) * C.astype(dtype)
    return R


def closed_gemm_exact(alpha, A, B, beta, C):
    """Exact rational result (tiny inputs only)."""
    fr = np.vectorize(lambda v: Fraction(float(v)) if not isinstance(v, (int, np.integer)) else Fraction(int(v)),
                      otypes=[object])
    R = Fraction(alpha) * fr(A).dot(fr(B))
    if beta != 0:
        R = R + Fraction(beta) * fr(C)
    return R


def rel_frobenius(got, want) -> float:
    want = np.asarray(want, dtype=np.longdouble)
    got = np.asarray(got, dtype=np.longdouble)
    den = np.sqrt((want * want).sum())
    num = np.sqrt(((got - want) ** 2).sum())
    return float(num / den) if den != 0 else float(num)


def closed_map2(op, a, b):
    """NumPy statement of the binary ops (single IEEE operation or integer ring operation per
    element, so bit-exact)."""
    name = op if isinstance(op, str) else {v: k for k, v in OP.items()}[op]
    with np.errstate(all="ignore"):
        if name == "add":
            return a + b
        if name == "sub":
            return a - b
        if name == "mul":
            return a * b
        if name == "div":
            if a.dtype.kind == "f":
                return a / b
            return _trunc_div(a, b)
        if name == "mod":
            return _trunc_mod(a, b)
        if name == "add_relu":
            t = a + b
            return np.where(0 >= t, np.zeros_like(t), t)
        if name == "add_sigmoid":
            t = a + b
            return (1 / (1 + np.exp(-t))).astype(a.dtype)
        if name == "add_tanh":
            return np.tanh(a + b).astype(a.dtype)
        if name == "relu_bwd":
            return np.where(a <= 0, np.zeros_like(b), b)
        if name == "max":
            return np.where(b <= a, a, b)
        if name == "min":
            return np.where(a <= b, a, b)
        if name == "sigmoid_bwd":
            return a * (1 - a) * b
        if name == "tanh_bwd":
            return b * (1 - a * a)
        if name == "sqdiff":
            return (a - b) * (a - b)
    raise KeyError(name)


def _trunc_div(a, b):
    """C / Nim `div`: truncation toward zero; x div 0 -> 0; min div -1 wraps to min."""
    info = np.iinfo(a.dtype)
    a, b = np.broadcast_arrays(a, b)
    out = np.zeros(a.shape, dtype=a.dtype)
    nz = b != 0
    safe_b = np.where(nz, b, 1)
    ovf = nz & (a == info.min) & (b == -1)
    safe_a = np.where(ovf, 0, a)
    q = np.abs(safe_a.astype(object)) // np.abs(safe_b.astype(object))
    sign = np.where((safe_a < 0) ^ (safe_b < 0), -1, 1).astype(object)
    out[...] = np.where(nz, (q * sign), 0).astype(a.dtype)
    out[ovf] = info.min
    return out


def _trunc_mod(a, b):
    a, b = np.broadcast_arrays(a, b)
    q = _trunc_div(a, b).astype(object)
    r = a.astype(object) - q * b.astype(object)
    r = np.where(b == 0, 0, r)
    info = np.iinfo(a.dtype)
    r = np.where((a == info.min) & (b == -1), 0, r)
    return r.astype(a.dtype)
