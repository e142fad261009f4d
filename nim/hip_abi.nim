## Raw `{.importc.}` binding of libam_hip.so (the C ABI of include/am_hip.h).
##
## This file is what a maintainer adds to Arraymancer (e.g. as
## src/arraymancer/tensor/backend/hip.nim) to reach the MI355X kernels; it takes the place of
## nimcuda + src/arraymancer/tensor/backend/{cuda,cublas,cuda_global_state}.nim.
##
## NOT COMPILED in the environment this repository is built in (no Nim toolchain there): every
## signature below is mechanically the one in include/am_hip.h, whose symbols and ctypes twins are
## checked by tests/test_abi.py.

const libAmHip* {.strdefine.} = "libam_hip.so"

{.push cdecl, dynlib: libAmHip.}

# ---- status codes
const
  AM_OK* = 0.cint
  AM_E_ARG* = -1.cint
  AM_E_SHAPE* = -2.cint
  AM_E_DTYPE* = -3.cint
  AM_E_ALLOC* = -4.cint
  AM_E_HIP* = -5.cint
  AM_E_NODEVICE* = -6.cint

# ---- runtime
proc am_hip_last_error*(): cstring {.importc.}
proc am_hip_version*(): cstring {.importc.}
proc am_hip_init*(device: cint): cint {.importc.}
proc am_hip_device_count*(count: ptr cint): cint {.importc.}
proc am_hip_device_info*(name: cstring, name_cap: csize_t, compute_units, clock_khz: ptr cint,
                         hbm_bytes: ptr csize_t, lds_bytes_per_cu: ptr cint): cint {.importc.}
proc am_hip_malloc*(bytes: csize_t, dptr: ptr pointer): cint {.importc.}
proc am_hip_empty_cache*(): cint {.importc.}   # freed blocks are cached for reuse; this returns them to the driver
proc am_hip_memory_stats*(live_bytes, cached_bytes: ptr csize_t): cint {.importc.}
proc am_hip_device_free_bytes*(free_bytes, total_bytes: ptr csize_t): cint {.importc.}
proc am_hip_free*(dptr: pointer): cint {.importc.}
proc am_hip_memcpy_h2d*(dst, src: pointer, bytes: csize_t): cint {.importc.}
proc am_hip_memcpy_d2h*(dst, src: pointer, bytes: csize_t): cint {.importc.}
proc am_hip_memcpy_d2d*(dst, src: pointer, bytes: csize_t): cint {.importc.}
proc am_hip_memset*(dst: pointer, byte_value: cint, bytes: csize_t): cint {.importc.}
proc am_hip_sync*(): cint {.importc.}
proc am_hip_stream*(): pointer {.importc.}
proc am_hip_event_create*(ev: ptr pointer): cint {.importc.}
proc am_hip_event_record*(ev: pointer): cint {.importc.}
proc am_hip_event_elapsed_ms*(start, stop: pointer, ms: ptr cfloat): cint {.importc.}
proc am_hip_event_destroy*(ev: pointer): cint {.importc.}

proc am_hip_graph_begin*(): cint {.importc.}
proc am_hip_alloc_hold*(on: cint): cint {.importc.}
proc am_hip_graph_end*(graph_exec: ptr pointer): cint {.importc.}
proc am_hip_graph_launch*(graph_exec: pointer): cint {.importc.}
proc am_hip_graph_destroy*(graph_exec: pointer): cint {.importc.}
proc am_hip_diag_peak*(kind, iters, waves_per_simd: cint, ops_per_second: ptr cdouble): cint {.importc.}
proc am_hip_diag_clock_begin*(): cint {.importc.}
proc am_hip_diag_clock_end*(shader_mhz: ptr cdouble): cint {.importc.}
proc am_hip_diag_phases_begin*(): cint {.importc.}
proc am_hip_diag_phases*(out6: ptr cdouble): cint {.importc.}
proc am_hip_diag_hbm*(kind: cint, bytes: csize_t, windows, blocks_per_cu, unroll, flags, launches: cint,
                      bytes_per_second: ptr cdouble): cint {.importc.}

# ---- GEMM (strides in elements; pointers already offset)
proc am_hip_gemm_f32*(M, N, K: int64, alpha: cfloat, A: ptr cfloat, rsA, csA: int64,
                      B: ptr cfloat, rsB, csB: int64, beta: cfloat,
                      C: ptr cfloat, rsC, csC: int64): cint {.importc.}
proc am_hip_gemm_noalloc_f32*(M, N, K: int64, alpha: cfloat, A: ptr cfloat, rsA, csA: int64,
                              B: ptr cfloat, rsB, csB: int64, beta: cfloat,
                              C: ptr cfloat, rsC, csC: int64): cint {.importc.}   # allocates nothing: split-K partials in a 16 MiB static device array
proc am_hip_gemm_f64*(M, N, K: int64, alpha: cdouble, A: ptr cdouble, rsA, csA: int64,
                      B: ptr cdouble, rsB, csB: int64, beta: cdouble,
                      C: ptr cdouble, rsC, csC: int64): cint {.importc.}
proc am_hip_gemm_i32*(M, N, K: int64, alpha: int32, A: ptr int32, rsA, csA: int64,
                      B: ptr int32, rsB, csB: int64, beta: int32,
                      C: ptr int32, rsC, csC: int64): cint {.importc.}
proc am_hip_gemm_i64*(M, N, K: int64, alpha: int64, A: ptr int64, rsA, csA: int64,
                      B: ptr int64, rsB, csB: int64, beta: int64,
                      C: ptr int64, rsC, csC: int64): cint {.importc.}

proc am_hip_digits_prepare_i32*(side: cint, rows, cols: int64, X: ptr int32, rs, cs: int64, handle: ptr pointer): cint {.importc.}
proc am_hip_digits_prepare_i64*(side: cint, rows, cols: int64, X: ptr int64, rs, cs: int64, handle: ptr pointer): cint {.importc.}
proc am_hip_digits_release*(handle: pointer): cint {.importc.}
proc am_hip_gemm_prepared_i32*(M, N, K: int64, alpha: int32, A: ptr int32, rsA, csA: int64, A_digits: pointer,
                               B: ptr int32, rsB, csB: int64, B_digits: pointer, beta: int32,
                               C: ptr int32, rsC, csC: int64): cint {.importc.}
proc am_hip_gemm_prepared_i64*(M, N, K: int64, alpha: int64, A: ptr int64, rsA, csA: int64, A_digits: pointer,
                               B: ptr int64, rsB, csB: int64, B_digits: pointer, beta: int64,
                               C: ptr int64, rsC, csC: int64): cint {.importc.}

proc am_hip_gemm_batched_f32*(batch, M, N, K: int64, alpha: cfloat, A: ptr cfloat, rsA, csA, bsA: int64,
                              B: ptr cfloat, rsB, csB, bsB: int64, beta: cfloat, C: ptr cfloat, rsC, csC, bsC: int64,
                              epilogue: cint, bias: ptr cfloat, bias_rs, bias_cs: int64): cint {.importc.}
proc am_hip_im2col_f32*(N: int64, C, H, W, kH, kW, padH, padW, strideH, strideW: cint, inp: ptr cfloat,
                        in_n, in_c, in_h, in_w: int64, col: ptr cfloat): cint {.importc.}
proc am_hip_im2col_strided_f32*(N: int64, C, H, W, kH, kW, padH, padW, strideH, strideW: cint, inp: ptr cfloat,
                                in_n, in_c, in_h, in_w: int64, col: ptr cfloat, col_n, col_c: int64): cint {.importc.}
proc am_hip_col2im_f32*(N: int64, C, H, W, kH, kW, padH, padW, strideH, strideW: cint, col: ptr cfloat,
                        col_n, col_c: int64, output: ptr cfloat, out_n, out_c, out_h, out_w: int64): cint {.importc.}
proc am_hip_gemm_batched_f64*(batch, M, N, K: int64, alpha: cdouble, A: ptr cdouble, rsA, csA, bsA: int64,
                              B: ptr cdouble, rsB, csB, bsB: int64, beta: cdouble, C: ptr cdouble, rsC, csC, bsC: int64,
                              epilogue: cint, bias: ptr cdouble, bias_rs, bias_cs: int64): cint {.importc.}
proc am_hip_im2col_f64*(N: int64, C, H, W, kH, kW, padH, padW, strideH, strideW: cint, inp: ptr cdouble,
                        in_n, in_c, in_h, in_w: int64, col: ptr cdouble): cint {.importc.}
proc am_hip_im2col_strided_f64*(N: int64, C, H, W, kH, kW, padH, padW, strideH, strideW: cint, inp: ptr cdouble,
                                in_n, in_c, in_h, in_w: int64, col: ptr cdouble, col_n, col_c: int64): cint {.importc.}
proc am_hip_col2im_f64*(N: int64, C, H, W, kH, kW, padH, padW, strideH, strideW: cint, col: ptr cdouble,
                        col_n, col_c: int64, output: ptr cdouble, out_n, out_c, out_h, out_w: int64): cint {.importc.}
proc am_hip_conv2d_f32*(N: int64, C, H, W, Cout, kH, kW, padH, padW, strideH, strideW: cint, inp: ptr cfloat,
                        in_n, in_c, in_h, in_w: int64, kernel: ptr cfloat, kernel_rs: int64, epilogue: cint,
                        bias: ptr cfloat, bias_s: int64, output: ptr cfloat): cint {.importc.}
proc am_hip_conv2d_f64*(N: int64, C, H, W, Cout, kH, kW, padH, padW, strideH, strideW: cint, inp: ptr cdouble,
                        in_n, in_c, in_h, in_w: int64, kernel: ptr cdouble, kernel_rs: int64, epilogue: cint,
                        bias: ptr cdouble, bias_s: int64, output: ptr cdouble): cint {.importc.}
proc am_hip_conv2d_grad_weight_f32*(N: int64, C, H, W, Cout, kH, kW, padH, padW, strideH, strideW: cint, inp: ptr cfloat,
                                    in_n, in_c, in_h, in_w: int64, grad_output: ptr cfloat, gout_rs: int64,
                                    output: ptr cfloat): cint {.importc.}
proc am_hip_conv2d_grad_weight_f64*(N: int64, C, H, W, Cout, kH, kW, padH, padW, strideH, strideW: cint, inp: ptr cdouble,
                                    in_n, in_c, in_h, in_w: int64, grad_output: ptr cdouble, gout_rs: int64,
                                    output: ptr cdouble): cint {.importc.}
proc am_hip_gemm_batched_i32*(batch, M, N, K: int64, alpha: int32, A: ptr int32, rsA, csA, bsA: int64,
                              B: ptr int32, rsB, csB, bsB: int64, beta: int32, C: ptr int32, rsC, csC, bsC: int64,
                              epilogue: cint, bias: ptr int32, bias_rs, bias_cs: int64): cint {.importc.}
proc am_hip_im2col_i32*(N: int64, C, H, W, kH, kW, padH, padW, strideH, strideW: cint, inp: ptr int32,
                        in_n, in_c, in_h, in_w: int64, col: ptr int32): cint {.importc.}
proc am_hip_im2col_strided_i32*(N: int64, C, H, W, kH, kW, padH, padW, strideH, strideW: cint, inp: ptr int32,
                                in_n, in_c, in_h, in_w: int64, col: ptr int32, col_n, col_c: int64): cint {.importc.}
proc am_hip_col2im_i32*(N: int64, C, H, W, kH, kW, padH, padW, strideH, strideW: cint, col: ptr int32,
                        col_n, col_c: int64, output: ptr int32, out_n, out_c, out_h, out_w: int64): cint {.importc.}
proc am_hip_gemm_batched_i64*(batch, M, N, K: int64, alpha: int64, A: ptr int64, rsA, csA, bsA: int64,
                              B: ptr int64, rsB, csB, bsB: int64, beta: int64, C: ptr int64, rsC, csC, bsC: int64,
                              epilogue: cint, bias: ptr int64, bias_rs, bias_cs: int64): cint {.importc.}
proc am_hip_im2col_i64*(N: int64, C, H, W, kH, kW, padH, padW, strideH, strideW: cint, inp: ptr int64,
                        in_n, in_c, in_h, in_w: int64, col: ptr int64): cint {.importc.}
proc am_hip_im2col_strided_i64*(N: int64, C, H, W, kH, kW, padH, padW, strideH, strideW: cint, inp: ptr int64,
                                in_n, in_c, in_h, in_w: int64, col: ptr int64, col_n, col_c: int64): cint {.importc.}
proc am_hip_col2im_i64*(N: int64, C, H, W, kH, kW, padH, padW, strideH, strideW: cint, col: ptr int64,
                        col_n, col_c: int64, output: ptr int64, out_n, out_c, out_h, out_w: int64): cint {.importc.}
proc am_hip_gemv_f32*(M, N: int64, alpha: cfloat, A: ptr cfloat, rsA, csA: int64, x: ptr cfloat, incx: int64,
                      beta: cfloat, y: ptr cfloat, incy: int64): cint {.importc.}
proc am_hip_gemv_f64*(M, N: int64, alpha: cdouble, A: ptr cdouble, rsA, csA: int64, x: ptr cdouble, incx: int64,
                      beta: cdouble, y: ptr cdouble, incy: int64): cint {.importc.}
proc am_hip_gemv_i32*(M, N: int64, alpha: int32, A: ptr int32, rsA, csA: int64, x: ptr int32, incx: int64,
                      beta: int32, y: ptr int32, incy: int64): cint {.importc.}
proc am_hip_gemv_i64*(M, N: int64, alpha: int64, A: ptr int64, rsA, csA: int64, x: ptr int64, incx: int64,
                      beta: int64, y: ptr int64, incy: int64): cint {.importc.}
proc am_hip_dot_f32*(n: int64, x: ptr cfloat, incx: int64, y: ptr cfloat, incy: int64, res: ptr cfloat): cint {.importc.}
proc am_hip_dot_f64*(n: int64, x: ptr cdouble, incx: int64, y: ptr cdouble, incy: int64, res: ptr cdouble): cint {.importc.}
proc am_hip_dot_i32*(n: int64, x: ptr int32, incx: int64, y: ptr int32, incy: int64, res: ptr int32): cint {.importc.}
proc am_hip_dot_i64*(n: int64, x: ptr int64, incx: int64, y: ptr int64, incy: int64, res: ptr int64): cint {.importc.}

# reductions, softmax, pooling — reduce_axis_inline / reduce_inline (higher_order_foldreduce.nim:22-61),
# softmax (nn_primitives/nnp_softmax.nim:18-38), maxpool2d (nn_primitives/nnp_maxpooling.nim:19-66)
const
  AM_RED_SUM* = 0.cint
  AM_RED_PROD* = 1.cint
  AM_RED_MIN* = 2.cint
  AM_RED_MAX* = 3.cint
proc am_hip_argreduce_f32*(op, rank: cint, shape: ptr int64, axis: cint, idx: ptr int64, idx_strides: ptr int64, val: ptr cfloat, val_strides: ptr int64, a: ptr cfloat, a_strides: ptr int64): cint {.importc.}
proc am_hip_argreduce_f64*(op, rank: cint, shape: ptr int64, axis: cint, idx: ptr int64, idx_strides: ptr int64, val: ptr cdouble, val_strides: ptr int64, a: ptr cdouble, a_strides: ptr int64): cint {.importc.}
proc am_hip_argreduce_i32*(op, rank: cint, shape: ptr int64, axis: cint, idx: ptr int64, idx_strides: ptr int64, val: ptr int32, val_strides: ptr int64, a: ptr int32, a_strides: ptr int64): cint {.importc.}
proc am_hip_argreduce_i64*(op, rank: cint, shape: ptr int64, axis: cint, idx: ptr int64, idx_strides: ptr int64, val: ptr int64, val_strides: ptr int64, a: ptr int64, a_strides: ptr int64): cint {.importc.}
proc am_hip_reduce_axis_f32*(op, rank: cint, shape: ptr int64, axis: cint, dst: ptr cfloat, dst_strides: ptr int64, a: ptr cfloat, a_strides: ptr int64): cint {.importc.}
proc am_hip_reduce_axis_f64*(op, rank: cint, shape: ptr int64, axis: cint, dst: ptr cdouble, dst_strides: ptr int64, a: ptr cdouble, a_strides: ptr int64): cint {.importc.}
proc am_hip_reduce_axis_i32*(op, rank: cint, shape: ptr int64, axis: cint, dst: ptr int32, dst_strides: ptr int64, a: ptr int32, a_strides: ptr int64): cint {.importc.}
proc am_hip_reduce_axis_i64*(op, rank: cint, shape: ptr int64, axis: cint, dst: ptr int64, dst_strides: ptr int64, a: ptr int64, a_strides: ptr int64): cint {.importc.}
proc am_hip_reduce_all_f32*(op, rank: cint, shape: ptr int64, a: ptr cfloat, a_strides: ptr int64, res: ptr cfloat): cint {.importc.}
proc am_hip_reduce_all_f64*(op, rank: cint, shape: ptr int64, a: ptr cdouble, a_strides: ptr int64, res: ptr cdouble): cint {.importc.}
proc am_hip_reduce_all_i32*(op, rank: cint, shape: ptr int64, a: ptr int32, a_strides: ptr int64, res: ptr int32): cint {.importc.}
proc am_hip_reduce_all_i64*(op, rank: cint, shape: ptr int64, a: ptr int64, a_strides: ptr int64, res: ptr int64): cint {.importc.}
proc am_hip_softmax_rows_f32*(rows, cols: int64, dst: ptr cfloat, dst_rs, dst_cs: int64, src: ptr cfloat, src_rs, src_cs: int64): cint {.importc.}
proc am_hip_softmax_rows_f64*(rows, cols: int64, dst: ptr cdouble, dst_rs, dst_cs: int64, src: ptr cdouble, src_rs, src_cs: int64): cint {.importc.}
proc am_hip_gru_gates_f32*(batch, H: int64, w3x: ptr cfloat, ldw: int64, u3h: ptr cfloat, ldu: int64, hidden: ptr cfloat, ldh: int64, r, z, n, uh: ptr cfloat, lds: int64): cint {.importc.}
proc am_hip_gru_gates_f64*(batch, H: int64, w3x: ptr cdouble, ldw: int64, u3h: ptr cdouble, ldu: int64, hidden: ptr cdouble, ldh: int64, r, z, n, uh: ptr cdouble, lds: int64): cint {.importc.}
proc am_hip_gru_gates_backward_f32*(batch, H: int64, dnext, h, r, z, n, uh: ptr cfloat, ld_in: int64, dw3x: ptr cfloat, ldw: int64, du3h: ptr cfloat, ldu: int64): cint {.importc.}
proc am_hip_gru_gates_backward_f64*(batch, H: int64, dnext, h, r, z, n, uh: ptr cdouble, ld_in: int64, dw3x: ptr cdouble, ldw: int64, du3h: ptr cdouble, ldu: int64): cint {.importc.}
proc am_hip_sgd_update_f32*(count: cint, values: ptr ptr cfloat, grads: ptr ptr cfloat, sizes: ptr int64, learning_rate: cfloat): cint {.importc.}
proc am_hip_sgd_update_f64*(count: cint, values: ptr ptr cdouble, grads: ptr ptr cdouble, sizes: ptr int64, learning_rate: cdouble): cint {.importc.}
proc am_hip_sigmoid_cross_entropy_f32*(rows, cols: int64, input: ptr cfloat, in_rs, in_cs: int64, target: ptr cfloat, t_rs, t_cs: int64, loss: ptr cfloat): cint {.importc.}
proc am_hip_sigmoid_cross_entropy_backward_f32*(rows, cols: int64, gradient: cfloat, input: ptr cfloat, in_rs, in_cs: int64, target: ptr cfloat, t_rs, t_cs: int64, res: ptr cfloat, r_rs, r_cs: int64): cint {.importc.}
proc am_hip_sigmoid_cross_entropy_f64*(rows, cols: int64, input: ptr cdouble, in_rs, in_cs: int64, target: ptr cdouble, t_rs, t_cs: int64, loss: ptr cdouble): cint {.importc.}
proc am_hip_sigmoid_cross_entropy_backward_f64*(rows, cols: int64, gradient: cdouble, input: ptr cdouble, in_rs, in_cs: int64, target: ptr cdouble, t_rs, t_cs: int64, res: ptr cdouble, r_rs, r_cs: int64): cint {.importc.}
proc am_hip_softmax_cross_entropy_f32*(rows, cols: int64, input: ptr cfloat, in_rs, in_cs: int64, target: ptr cfloat, t_rs, t_cs: int64, loss: ptr cfloat): cint {.importc.}
proc am_hip_sparse_softmax_cross_entropy_f32*(rows, cols: int64, input: ptr cfloat, in_rs, in_cs: int64, labels: ptr int64, labels_s: int64, loss: ptr cfloat): cint {.importc.}
proc am_hip_softmax_cross_entropy_backward_f32*(rows, cols: int64, gradient: cfloat, input: ptr cfloat, in_rs, in_cs: int64, target: ptr cfloat, t_rs, t_cs: int64, res: ptr cfloat, r_rs, r_cs: int64): cint {.importc.}
proc am_hip_sparse_softmax_cross_entropy_backward_f32*(rows, cols: int64, gradient: cfloat, input: ptr cfloat, in_rs, in_cs: int64, labels: ptr int64, labels_s: int64, res: ptr cfloat, r_rs, r_cs: int64): cint {.importc.}
proc am_hip_softmax_cross_entropy_f64*(rows, cols: int64, input: ptr cdouble, in_rs, in_cs: int64, target: ptr cdouble, t_rs, t_cs: int64, loss: ptr cdouble): cint {.importc.}
proc am_hip_sparse_softmax_cross_entropy_f64*(rows, cols: int64, input: ptr cdouble, in_rs, in_cs: int64, labels: ptr int64, labels_s: int64, loss: ptr cdouble): cint {.importc.}
proc am_hip_softmax_cross_entropy_backward_f64*(rows, cols: int64, gradient: cdouble, input: ptr cdouble, in_rs, in_cs: int64, target: ptr cdouble, t_rs, t_cs: int64, res: ptr cdouble, r_rs, r_cs: int64): cint {.importc.}
proc am_hip_sparse_softmax_cross_entropy_backward_f64*(rows, cols: int64, gradient: cdouble, input: ptr cdouble, in_rs, in_cs: int64, labels: ptr int64, labels_s: int64, res: ptr cdouble, r_rs, r_cs: int64): cint {.importc.}
proc am_hip_maxpool2d_backward_f32*(N: int64, C, H, W, kH, kW, padH, padW, strideH, strideW: cint, argmax: ptr int64, grad_output: ptr cfloat, grad_input: ptr cfloat): cint {.importc.}
proc am_hip_maxpool2d_backward_f64*(N: int64, C, H, W, kH, kW, padH, padW, strideH, strideW: cint, argmax: ptr int64, grad_output: ptr cdouble, grad_input: ptr cdouble): cint {.importc.}
proc am_hip_maxpool2d_backward_i32*(N: int64, C, H, W, kH, kW, padH, padW, strideH, strideW: cint, argmax: ptr int64, grad_output: ptr int32, grad_input: ptr int32): cint {.importc.}
proc am_hip_maxpool2d_backward_i64*(N: int64, C, H, W, kH, kW, padH, padW, strideH, strideW: cint, argmax: ptr int64, grad_output: ptr int64, grad_input: ptr int64): cint {.importc.}
proc am_hip_maxpool2d_f32*(N: int64, C, H, W, kH, kW, padH, padW, strideH, strideW: cint, inp: ptr cfloat, outp: ptr cfloat, argmax: ptr int64): cint {.importc.}
proc am_hip_maxpool2d_f64*(N: int64, C, H, W, kH, kW, padH, padW, strideH, strideW: cint, inp: ptr cdouble, outp: ptr cdouble, argmax: ptr int64): cint {.importc.}
proc am_hip_maxpool2d_i32*(N: int64, C, H, W, kH, kW, padH, padW, strideH, strideW: cint, inp: ptr int32, outp: ptr int32, argmax: ptr int64): cint {.importc.}
proc am_hip_maxpool2d_i64*(N: int64, C, H, W, kH, kW, padH, padW, strideH, strideW: cint, inp: ptr int64, outp: ptr int64, argmax: ptr int64): cint {.importc.}

const
  AM_EPI_NONE* = 0.cint
  AM_EPI_BIAS* = 1.cint
  AM_EPI_RELU* = 2.cint
  AM_EPI_BIAS_RELU* = 3.cint

proc am_hip_gemm_ex_f32*(M, N, K: int64, alpha: cfloat, A: ptr cfloat, rsA, csA: int64,
                         B: ptr cfloat, rsB, csB: int64, beta: cfloat,
                         C: ptr cfloat, rsC, csC: int64,
                         epilogue: cint, bias: ptr cfloat, bias_rs, bias_cs: int64): cint {.importc.}
proc am_hip_gemm_ex_f64*(M, N, K: int64, alpha: cdouble, A: ptr cdouble, rsA, csA: int64,
                         B: ptr cdouble, rsB, csB: int64, beta: cdouble,
                         C: ptr cdouble, rsC, csC: int64,
                         epilogue: cint, bias: ptr cdouble, bias_rs, bias_cs: int64): cint {.importc.}

# ---- element-wise / broadcast / map
type
  AmBinaryOp* {.size: sizeof(cint).} = enum
    opAdd = 0, opSub = 1, opMul = 2, opDiv = 3, opMod = 4, opAddRelu = 5, opAddSigmoid = 6,
    opAddTanh = 7, opReluBwd = 8, opMax = 9, opMin = 10, opSigmoidBwd = 11, opTanhBwd = 12, opSqDiff = 13,
    opPow = 14, opFloorMod = 15, opCopySign = 16
  AmCompareOp* {.size: sizeof(cint).} = enum   # results are Tensor[bool]: one byte per element
    cmpEq = 0, cmpNe = 1, cmpLt = 2, cmpLe = 3, cmpGt = 4, cmpGe = 5, cmpModIsZero = 6
  AmPredicate* {.size: sizeof(cint).} = enum
    predIsNaN = 0, predIsNotNaN = 1, predClassify = 2
  AmUnaryOp* {.size: sizeof(cint).} = enum
    uopCopy = 0, uopNeg = 1, uopRelu = 2, uopSigmoid = 3, uopTanh = 4, uopExp = 5, uopAbs = 6, uopSqrt = 7, uopSquare = 8,
    uopLn = 9, uopLog10 = 10, uopLog2 = 11, uopSin = 12, uopCos = 13, uopTan = 14, uopSinh = 15, uopCosh = 16,
    uopArcsin = 17, uopArccos = 18, uopArctan = 19, uopArcsinh = 20, uopArccosh = 21, uopArctanh = 22, uopCbrt = 23,
    uopErf = 24, uopErfc = 25, uopGamma = 26, uopLgamma = 27, uopFloor = 28, uopCeil = 29, uopTrunc = 30,
    uopRound = 31, uopReciprocal = 32, uopDegToRad = 33, uopRadToDeg = 34, uopFac = 35

proc am_hip_ew_binary_f32*(op: cint, rank: cint, shape: ptr int64, dst: ptr cfloat, dst_strides: ptr int64,
                           a: ptr cfloat, a_strides: ptr int64, b: ptr cfloat, b_strides: ptr int64): cint {.importc.}
proc am_hip_ew_binary_f64*(op: cint, rank: cint, shape: ptr int64, dst: ptr cdouble, dst_strides: ptr int64,
                           a: ptr cdouble, a_strides: ptr int64, b: ptr cdouble, b_strides: ptr int64): cint {.importc.}
proc am_hip_ew_binary_i32*(op: cint, rank: cint, shape: ptr int64, dst: ptr int32, dst_strides: ptr int64,
                           a: ptr int32, a_strides: ptr int64, b: ptr int32, b_strides: ptr int64): cint {.importc.}
proc am_hip_ew_binary_i64*(op: cint, rank: cint, shape: ptr int64, dst: ptr int64, dst_strides: ptr int64,
                           a: ptr int64, a_strides: ptr int64, b: ptr int64, b_strides: ptr int64): cint {.importc.}

proc am_hip_ew_scalar_f32*(op, scalar_on_left, rank: cint, shape: ptr int64, dst: ptr cfloat, dst_strides: ptr int64,
                           a: ptr cfloat, a_strides: ptr int64, scalar: cfloat): cint {.importc.}
proc am_hip_ew_scalar_f64*(op, scalar_on_left, rank: cint, shape: ptr int64, dst: ptr cdouble, dst_strides: ptr int64,
                           a: ptr cdouble, a_strides: ptr int64, scalar: cdouble): cint {.importc.}
proc am_hip_ew_scalar_i32*(op, scalar_on_left, rank: cint, shape: ptr int64, dst: ptr int32, dst_strides: ptr int64,
                           a: ptr int32, a_strides: ptr int64, scalar: int32): cint {.importc.}
proc am_hip_ew_scalar_i64*(op, scalar_on_left, rank: cint, shape: ptr int64, dst: ptr int64, dst_strides: ptr int64,
                           a: ptr int64, a_strides: ptr int64, scalar: int64): cint {.importc.}

proc am_hip_ew_ternary_f32*(op, rank: cint, shape: ptr int64, dst: ptr cfloat, dst_strides: ptr int64,
                            a: ptr cfloat, a_strides: ptr int64, b: ptr cfloat, b_strides: ptr int64,
                            c: ptr cfloat, c_strides: ptr int64): cint {.importc.}
proc am_hip_ew_ternary_f64*(op, rank: cint, shape: ptr int64, dst: ptr cdouble, dst_strides: ptr int64,
                            a: ptr cdouble, a_strides: ptr int64, b: ptr cdouble, b_strides: ptr int64,
                            c: ptr cdouble, c_strides: ptr int64): cint {.importc.}
proc am_hip_ew_ternary_i32*(op, rank: cint, shape: ptr int64, dst: ptr int32, dst_strides: ptr int64,
                            a: ptr int32, a_strides: ptr int64, b: ptr int32, b_strides: ptr int64,
                            c: ptr int32, c_strides: ptr int64): cint {.importc.}
proc am_hip_ew_ternary_i64*(op, rank: cint, shape: ptr int64, dst: ptr int64, dst_strides: ptr int64,
                            a: ptr int64, a_strides: ptr int64, b: ptr int64, b_strides: ptr int64,
                            c: ptr int64, c_strides: ptr int64): cint {.importc.}

proc am_hip_ew_unary_f32*(op, rank: cint, shape: ptr int64, dst: ptr cfloat, dst_strides: ptr int64,
                          a: ptr cfloat, a_strides: ptr int64): cint {.importc.}
proc am_hip_ew_unary_f64*(op, rank: cint, shape: ptr int64, dst: ptr cdouble, dst_strides: ptr int64,
                          a: ptr cdouble, a_strides: ptr int64): cint {.importc.}
proc am_hip_ew_unary_i32*(op, rank: cint, shape: ptr int64, dst: ptr int32, dst_strides: ptr int64,
                          a: ptr int32, a_strides: ptr int64): cint {.importc.}
proc am_hip_ew_unary_i64*(op, rank: cint, shape: ptr int64, dst: ptr int64, dst_strides: ptr int64,
                          a: ptr int64, a_strides: ptr int64): cint {.importc.}

# map bodies whose result type differs from the operands' (comparisons -> bool, sgn -> int), clamp with bounds by value
proc am_hip_ew_compare_f32*(op, rank: cint, shape: ptr int64, dst: ptr uint8, dst_strides: ptr int64,
                            a: ptr cfloat, a_strides: ptr int64, b: ptr cfloat, b_strides: ptr int64): cint {.importc.}
proc am_hip_ew_compare_f64*(op, rank: cint, shape: ptr int64, dst: ptr uint8, dst_strides: ptr int64,
                            a: ptr cdouble, a_strides: ptr int64, b: ptr cdouble, b_strides: ptr int64): cint {.importc.}
proc am_hip_ew_compare_i32*(op, rank: cint, shape: ptr int64, dst: ptr uint8, dst_strides: ptr int64,
                            a: ptr int32, a_strides: ptr int64, b: ptr int32, b_strides: ptr int64): cint {.importc.}
proc am_hip_ew_compare_i64*(op, rank: cint, shape: ptr int64, dst: ptr uint8, dst_strides: ptr int64,
                            a: ptr int64, a_strides: ptr int64, b: ptr int64, b_strides: ptr int64): cint {.importc.}
proc am_hip_ew_compare_scalar_f32*(op, rank: cint, shape: ptr int64, dst: ptr uint8, dst_strides: ptr int64,
                                   a: ptr cfloat, a_strides: ptr int64, scalar: cfloat): cint {.importc.}
proc am_hip_ew_compare_scalar_f64*(op, rank: cint, shape: ptr int64, dst: ptr uint8, dst_strides: ptr int64,
                                   a: ptr cdouble, a_strides: ptr int64, scalar: cdouble): cint {.importc.}
proc am_hip_ew_compare_scalar_i32*(op, rank: cint, shape: ptr int64, dst: ptr uint8, dst_strides: ptr int64,
                                   a: ptr int32, a_strides: ptr int64, scalar: int32): cint {.importc.}
proc am_hip_ew_compare_scalar_i64*(op, rank: cint, shape: ptr int64, dst: ptr uint8, dst_strides: ptr int64,
                                   a: ptr int64, a_strides: ptr int64, scalar: int64): cint {.importc.}
proc am_hip_ew_predicate_f32*(op, rank: cint, shape: ptr int64, dst: ptr uint8, dst_strides: ptr int64,
                              a: ptr cfloat, a_strides: ptr int64): cint {.importc.}
proc am_hip_ew_predicate_f64*(op, rank: cint, shape: ptr int64, dst: ptr uint8, dst_strides: ptr int64,
                              a: ptr cdouble, a_strides: ptr int64): cint {.importc.}
proc am_hip_ew_sgn_f32*(rank: cint, shape: ptr int64, dst: ptr int64, dst_strides: ptr int64,
                        a: ptr cfloat, a_strides: ptr int64): cint {.importc.}
proc am_hip_ew_sgn_f64*(rank: cint, shape: ptr int64, dst: ptr int64, dst_strides: ptr int64,
                        a: ptr cdouble, a_strides: ptr int64): cint {.importc.}
proc am_hip_ew_sgn_i32*(rank: cint, shape: ptr int64, dst: ptr int64, dst_strides: ptr int64,
                        a: ptr int32, a_strides: ptr int64): cint {.importc.}
proc am_hip_ew_sgn_i64*(rank: cint, shape: ptr int64, dst: ptr int64, dst_strides: ptr int64,
                        a: ptr int64, a_strides: ptr int64): cint {.importc.}
proc am_hip_ew_clamp_f32*(rank: cint, shape: ptr int64, dst: ptr cfloat, dst_strides: ptr int64,
                          a: ptr cfloat, a_strides: ptr int64, lo, hi: cfloat): cint {.importc.}
proc am_hip_ew_clamp_f64*(rank: cint, shape: ptr int64, dst: ptr cdouble, dst_strides: ptr int64,
                          a: ptr cdouble, a_strides: ptr int64, lo, hi: cdouble): cint {.importc.}
proc am_hip_ew_clamp_i32*(rank: cint, shape: ptr int64, dst: ptr int32, dst_strides: ptr int64,
                          a: ptr int32, a_strides: ptr int64, lo, hi: int32): cint {.importc.}
proc am_hip_ew_clamp_i64*(rank: cint, shape: ptr int64, dst: ptr int64, dst_strides: ptr int64,
                          a: ptr int64, a_strides: ptr int64, lo, hi: int64): cint {.importc.}

{.pop.}

# ---- status -> exception, the role of nimcuda's `check` (src/arraymancer/tensor/backend/cuda.nim:27)
type HipError* = object of CatchableError

proc check*(rc: cint) {.inline.} =
  if rc == AM_OK: return
  let msg = $am_hip_last_error()
  case rc
  of AM_E_ARG, AM_E_SHAPE: raise newException(ValueError, msg)
  of AM_E_DTYPE: raise newException(ValueError, msg)
  of AM_E_ALLOC: raise newException(OutOfMemDefect, msg)
  else: raise newException(HipError, msg)
