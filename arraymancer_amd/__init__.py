"""arraymancer_amd — MI355X (gfx950) backend for Arraymancer's GEMM + broadcast/map hot path.

The product is the HIP library behind include/am_hip.h (arraymancer_amd/libam_hip.so, built by
`python -m arraymancer_amd.build`); this package is its host-side mirror of the reference's GPU
tensor backend. Importing the package does not load the library; the first device operation
does, and raises if it is missing (there is no CPU fallback).
"""
from ._lib import HipAllocError, HipError, load as load_library
from .metadata import Layout, Step
from .io_npy import read_npy, write_npy
from .tensor_hip import (OPERATORS, Graph, DigitPlanes, digits_prepare, HipStorage, HipTensor, apply2, apply3, map3, bc_add, bc_div, bc_mod, bc_mul,
                         bc_sub, bias_relu, conv2d, conv2d_into, conv2d_backward, col2im, im2col_folded, dot, empty, gemm, gemm_batched, gemv, im2col, linear, map2, matmul, relu, scalar_op,
                         sigmoid, sync, toHip, broadcast, unary, zeros, reduce_axis, reduce_all, tsum as sum, tproduct as product,
                         tmin as min, tmax as max, mean, softmax, softmax_cross_entropy, sparse_softmax_cross_entropy,
                         softmax_cross_entropy_backward, sparse_softmax_cross_entropy_backward, sigmoid_cross_entropy,
                         sigmoid_cross_entropy_backward, maxpool2d, tanh, relu_backward, sigmoid_backward,
                         tanh_backward, linear_backward, gru_cell_inference, gru_cell_forward, gru_cell_backward, gru_inference, gru_forward, gru_backward, variance, std, sqrt, square, argmax_max, argmax,
                         argmin_min, argmin, maxpool2d_backward, bc_pow, mreciprocal, clamp, mclamp, UFUNCS, ln, log10, log2, exp,
                         cbrt, sin, cos, tan, sinh, cosh, arcsin, arccos, arctan, arcsinh, arccosh, arctanh, erf, erfc,
                         gamma, lgamma, floor, ceil, trunc, reciprocal, tround as round, bc_eq, bc_ne, bc_lt, bc_le, bc_gt,
                         bc_ge, isNaN, isNotNaN, classify, FLOAT_CLASS, sgn, floorMod, copySign, mcopySign, degToRad, radToDeg, fac, sgd_update)

__all__ = [
    "HipTensor", "HipStorage", "Graph", "DigitPlanes", "digits_prepare", "HipError", "HipAllocError", "Layout", "Step", "OPERATORS",
    "toHip", "broadcast", "empty", "zeros", "sync", "gemm", "gemm_batched", "gemv", "dot", "im2col", "im2col_folded", "col2im", "conv2d", "conv2d_into", "conv2d_backward", "matmul", "linear", "map2", "apply2", "map3", "apply3", "scalar_op",
    "unary", "relu", "sigmoid", "bias_relu", "bc_add", "bc_sub", "bc_mul", "bc_div", "bc_mod",
    "tanh", "relu_backward", "sigmoid_backward", "tanh_backward", "linear_backward", "gru_cell_inference", "gru_cell_forward", "gru_cell_backward", "gru_inference", "gru_forward", "gru_backward",
    "variance", "std", "sqrt", "square", "argmax_max", "argmax", "argmin_min", "argmin", "maxpool2d_backward",
    "reduce_axis", "reduce_all", "sum", "product", "min", "max", "mean", "softmax", "maxpool2d", "softmax_cross_entropy", "sparse_softmax_cross_entropy",
    "softmax_cross_entropy_backward", "sparse_softmax_cross_entropy_backward", "sigmoid_cross_entropy", "sigmoid_cross_entropy_backward",
    "bc_pow", "mreciprocal", "clamp", "mclamp", "UFUNCS", "ln", "log10", "log2", "exp", "cbrt", "sin", "cos", "tan", "sinh", "cosh",
    "arcsin", "arccos", "arctan", "arcsinh", "arccosh", "arctanh", "erf", "erfc", "gamma", "lgamma", "floor", "ceil",
    "trunc", "reciprocal", "round",
    "bc_eq", "bc_ne", "bc_lt", "bc_le", "bc_gt", "bc_ge", "isNaN", "isNotNaN", "classify", "FLOAT_CLASS", "sgn", "floorMod",
    "copySign", "mcopySign", "degToRad", "radToDeg", "fac", "sgd_update",
    "read_npy", "write_npy", "load_library",
]
