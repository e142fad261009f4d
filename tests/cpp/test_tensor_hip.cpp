// C++ twin of the reference's GPU-backend unit tests, driven through am::HipTensor
// (include/am_hip_tensor.hpp) and therefore through the C ABI. Literals are the ones of
//   tests/tensor/test_operators_blas_cuda.nim, tests/tensor/test_broadcasting_cuda.nim,
//   tests/tensor/test_operators_blas.nim (integer cases, strided slices),
//   src/arraymancer/laser/primitives/matrix_multiplication/gemm.nim:315-567.
// Exit code 0 = every check passed. Needs an MI355X; run by tests/test_cpp_host_gpu.py.
#include <cmath>
#include <cstdio>
#include <fstream>
#include <iterator>
#include <string>
#include <vector>

#include "am_hip_tensor.hpp"

using am::HipTensor;
using am::Shape;
using am::toHip;

static int g_failed = 0, g_checked = 0;
#define CHECK(cond)                                                          \
  do {                                                                       \
    ++g_checked;                                                             \
    if (!(cond)) { ++g_failed; std::printf("FAILED %s:%d  %s\n", __FILE__, __LINE__, #cond); } \
  } while (0)
#define EXPECT_THROW(expr, EXC)                                              \
  do {                                                                       \
    ++g_checked;                                                             \
    bool ok_ = false;                                                        \
    try { (void)(expr); } catch (const EXC&) { ok_ = true; } catch (...) {}  \
    if (!ok_) { ++g_failed; std::printf("FAILED %s:%d  %s did not throw %s\n", __FILE__, __LINE__, #expr, #EXC); } \
  } while (0)

template <typename T>
static bool eq(const HipTensor<T>& t, const std::vector<T>& want) { return t.toCpu() == want; }

template <typename T>
static void gemm_literals() {
  // gemm.nim:373-396 / test_operators_blas_cuda.nim:19-35
  auto a = toHip<T>({1, 2, 3, 4, 5, 6}, {2, 3});
  auto b = toHip<T>({7, 8, 9, 10, 11, 12}, {3, 2});
  CHECK(eq(a * b, {58, 64, 139, 154}));
  // (M x K) * (K x N) with M < N, gemm.nim:398-422
  auto u = toHip<T>({-2, -3, -1, 3, 0, 4}, {2, 3});
  auto v = toHip<T>({1, 5, 2, -1, -3, 0, 3, 4, 6, -2, 7, -4}, {3, 4});
  CHECK(eq(u * v, {1, -8, -20, -6, 27, 7, 34, -19}));
  // M > N, gemm.nim:424-453
  auto m1 = toHip<T>({5, 6, 5, 8, 8, 2, 8, 8, 0, 5, 4, 0, 4, 0, 5, 6, 4, 5, 0, 3}, {5, 4});
  auto m2 = toHip<T>({5, 3, 6, 0, 5, 2, 3, 3, 8, 8, 2, 0, 7, 7, 0, 0}, {4, 4});
  CHECK(eq(m1 * m2, {151, 123, 58, 18, 170, 148, 70, 6, 57, 42, 23, 15, 102, 94, 34, 0, 66, 43, 39, 15}));
  // transposed operands, test_operators_blas.nim:133-149
  auto at = toHip<T>({1, 4, 2, 5, 3, 6}, {3, 2});
  auto bt = toHip<T>({7, 9, 11, 8, 10, 12}, {2, 3});
  CHECK(eq(at.transpose() * b, {58, 64, 139, 154}));
  CHECK(eq(a * bt.transpose(), {58, 64, 139, 154}));
  CHECK(eq(at.transpose() * bt.transpose(), {58, 64, 139, 154}));
  // matrix * vector
  auto d = toHip<T>({1, -1, 2, 0, -3, 1}, {2, 3});
  auto e = toHip<T>({2, 1, 0}, {3});
  CHECK(eq(d * e, {1, -3}));
  // dimension mismatch -> IndexDefect in the reference (test_operators_blas_cuda.nim:100-104)
  EXPECT_THROW(a * a, std::out_of_range);
  EXPECT_THROW(e * a, std::invalid_argument);
  // gemm(alpha, A, B, beta, C) on a strided destination (every other column of a wider buffer)
  auto wide = toHip<T>(std::vector<T>(8, T(1)), {2, 4});
  auto cview = wide.slice(1, 0, 2, 2);
  am::gemm(T(2), a, b, T(3), cview);
  CHECK(eq(wide, {T(2 * 58 + 3), 1, T(2 * 64 + 3), 1, T(2 * 139 + 3), 1, T(2 * 154 + 3), 1}));
}

static void integer_slices() {
  // test_operators_blas.nim:332-365: non-contiguous slices with negative steps
  auto b = toHip<int64_t>({-87, 44, 13, 1, 8, -16, 8, 91, 6, -2, 56, -56, 82, 70, 34, 23, 52, -70, 0, 53, 35, 94, 39, 36}, {6, 4});
  auto u = toHip<int64_t>({-91, 81, 69, -75}, {4});
  CHECK(eq(b * u, {12303, -8297, 7356, -1171, -14377, 4420}));
  auto b2 = b.slice(0, 4, 2, -2).slice(1, 3, 1, -2);
  auto u2 = u.slice(0, 2, 0, -2);
  CHECK(eq(b2 * u2, {10027, -3682}));
  auto b3 = b.slice(0, 2, 3).slice(1, 3, 1, -2);
  CHECK(eq(b3 * u2, {-3682, -4783}));
  // dot, test_operators_blas.nim:195-201
  CHECK(am::dot(toHip<int64_t>({1, 3, -5}, {3}), toHip<int64_t>({4, -2, -1}, {3})) == 3);
  CHECK(am::dot(toHip<double>({1, 3, -5}, {3}), toHip<double>({4, -2, -1}, {3})) == 3.0);
  // wraparound
  auto w = toHip<int32_t>({2147483647, 1}, {1, 2});
  auto x = toHip<int32_t>({2, 3}, {2, 1});
  CHECK(eq(w * x, {1}));
}

static void add_sub_scalars() {
  // test_operators_blas_cuda.nim:121-247
  auto u = toHip<double>({1, 3, -5}, {3});
  auto v = toHip<double>({4, -2, -1}, {3});
  u += v;
  CHECK(eq(u, {5, 1, -6}));
  u -= v;
  CHECK(eq(u + v, {5, 1, -6}) && eq(u - v, {-3, 5, -4}));
  auto t = toHip<float>({1, 1, 1, 2, 4, 8, 3, 9, 27}, {3, 3});
  auto z = t.clone().transpose();
  z += z;
  CHECK(eq(z, {2, 4, 6, 2, 8, 18, 2, 16, 54}));
  z += t;
  CHECK(eq(z, {3, 5, 7, 4, 12, 26, 5, 25, 81}));
  EXPECT_THROW(z += t.slice(0, 0, 1).slice(1, 0, 1), std::invalid_argument);
  auto a = toHip<double>({1, 2, 3, 4, 5, 6, 7, 8, 9}, {3, 3});
  auto a_t = a.transpose();
  CHECK(eq(a.slice(0, 0, 1).slice(1, 0, 1) + a_t.slice(0, 0, 1).slice(1, 0, 1), {2, 6, 6, 10}));
  CHECK(eq(a.slice(0, 1, 2).slice(1, 1, 2) - a_t.slice(0, 1, 2).slice(1, 1, 2), {0, -2, 2, 0}));
  auto s = toHip<double>({2, 6, -10}, {3});
  CHECK(eq(s / 2.0, {1, 3, -5}));
  auto f = toHip<float>({1, 3, -5}, {3});
  CHECK(eq(2.0f * f, {2, 6, -10}) && eq(f * 2.0f, {2, 6, -10}));
}

template <typename U>
static void unsigned_ring_ops() {
  // gemm.nim:275-307: unsigned element types ride the signed kernels. The small GEMM literals (gemm.nim:373-396) with
  // non-negative entries, then values whose sum and product leave the signed range: the ring's answer modulo 2^n.
  auto a = toHip<U>({1, 2, 3, 4, 5, 6}, {2, 3});
  auto b = toHip<U>({7, 8, 9, 10, 11, 12}, {3, 2});
  CHECK(eq(a * b, {58, 64, 139, 154}));
  const U top = U(1) << (8 * sizeof(U) - 1);             // 2^(n-1): the sign bit of the twin
  auto x = toHip<U>({top, U(top + 5), 3, U(~U(0))}, {2, 2});
  auto y = toHip<U>({2, 1, 1, 3}, {2, 2});
  // [[2*top + (top+5), top + 3*(top+5)], [6 + (2^n - 1), 3 + 3*(2^n - 1)]] modulo 2^n
  CHECK(eq(x * y, {U(top + 5), U(15), U(5), U(0)}));
  CHECK(eq(x + x, {U(0), U(10), U(6), U(~U(0) - 1)}));
  CHECK(eq(x - y, {U(top - 2), U(top + 4), U(2), U(~U(0) - 3)}));
  CHECK(eq(U(3) * x, {top, U(top + 15), U(9), U(~U(0) - 2)}));
  CHECK(am::sum(x) == U(U(2) * top + 5 + 3 + ~U(0)));
  CHECK(eq(am::broadcast(U(~U(0)), {2, 2}) + y, {U(1), U(0), U(0), U(2)}));   // scalar broadcast: strides 0, one element
  EXPECT_THROW(am::scalar_op(AM_OP_DIV, x, U(2)), std::invalid_argument);
  EXPECT_THROW(am::map2(AM_OP_MOD, x, y), std::invalid_argument);
  EXPECT_THROW(am::reduce_all(AM_RED_MAX, x), std::invalid_argument);
}

static void scalar_broadcast() {
  // broadcast(val, shape), shapeshifting.nim:136-176: one element of storage, every stride 0
  auto t = am::broadcast(2.5f, {3, 4});
  CHECK(t.storage->len == 1 && t.strides == Shape({0, 0}) && t.shape == Shape({3, 4}));
  CHECK(eq(t, std::vector<float>(12, 2.5f)));
  auto m = toHip<float>({1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12}, {3, 4});
  CHECK(eq(m + t, {3.5f, 4.5f, 5.5f, 6.5f, 7.5f, 8.5f, 9.5f, 10.5f, 11.5f, 12.5f, 13.5f, 14.5f}));
  CHECK(eq(am::broadcast(int64_t(-7), {2, 0, 3}), {}));
}

template <typename T>
static void broadcasting() {
  // test_broadcasting_cuda.nim:18-189 / test_broadcasting.nim:58-240
  auto a = toHip<T>({0, 10, 20, 30}, {4, 1});
  auto b = toHip<T>({0, 1, 2}, {1, 3});
  CHECK(eq(am::bc_add(a, b), {0, 1, 2, 10, 11, 12, 20, 21, 22, 30, 31, 32}));
  CHECK(eq(am::bc_sub(a, b), {0, -1, -2, 10, 9, 8, 20, 19, 18, 30, 29, 28}));
  CHECK(eq(am::bc_mul(a, b), {0, 0, 0, 0, 10, 20, 0, 20, 40, 0, 30, 60}));
  auto c = toHip<T>({100, 10, 20, 30}, {4, 1});
  auto d = toHip<T>({2, 5, 10}, {1, 3});
  CHECK(eq(am::bc_div(c, d), {50, 20, 10, 5, 2, 1, 10, 4, 2, 15, 6, 3}));
  auto e = a.broadcast({4, 3}).clone();
  e.bc_iadd(b);
  CHECK(eq(e, {0, 1, 2, 10, 11, 12, 20, 21, 22, 30, 31, 32}));
  e.bc_isub(b);
  e.bc_imul(b);
  CHECK(eq(e, {0, 0, 0, 0, 10, 20, 0, 20, 40, 0, 30, 60}));
  CHECK(eq(am::bc_add(am::bc_add(T(100), a), T(200)), {300, 310, 320, 330}));
  CHECK(eq(am::bc_sub(am::bc_sub(T(100), a), T(200)), {-100, -110, -120, -130}));
  CHECK(eq(am::bc_mul(am::bc_mul(T(10), a), T(20)), {0, 2000, 4000, 6000}));
  EXPECT_THROW(am::bc_add(toHip<T>(std::vector<T>(8, 0), {4, 2}), b), std::invalid_argument);
  // explicit broadcast, test_broadcasting.nim:39-56
  CHECK(eq(toHip<T>({2}, {1, 1}).broadcast({3, 2}).clone(), {2, 2, 2, 2, 2, 2}));
  CHECK(eq(toHip<T>({1, 2}, {2, 1}).broadcast({2, 2}), {1, 1, 2, 2}));
}

static void variance_std() {
  // tests/tensor/test_aggregate.nim:88-110
  auto a = toHip<double>({-3, -2, -1, 0, 1, 2, 3}, {7});
  CHECK(std::fabs(am::variance(a) - 4.6666666666667) < 1e-8);
  CHECK(std::fabs(am::stddev(a) - 2.1602468994693) < 1e-8);
  auto b = toHip<double>({1, 2, 3, -4, 0, 4, -2, 5}, {2, 4});
  CHECK(eq(am::variance(b, 0), {0.5, 2.0, 12.5, 40.5}));
  auto v1 = am::variance(b, 1).toCpu();
  CHECK(v1.size() == 2 && std::fabs(v1[0] - 9.666666666666666) + std::fabs(v1[1] - 10.91666666666667) < 1e-8);
  auto s0 = am::stddev(b, 0).toCpu();
  CHECK(std::fabs(s0[0] - 0.7071067811865476) + std::fabs(s0[3] - 6.363961030678928) < 1e-8);
  CHECK(eq(am::sqrt(toHip<float>({4, 9, 0.25f}, {3})), {2, 3, 0.5f}));
  CHECK(eq(am::square(toHip<int32_t>({-3, 65536, 7}, {3})), {9, 0, 49}));
}

static void pow_and_universal_functions() {
  // tests/tensor/test_broadcasting.nim:130-146, 340-362: `^.`, `^.=`
  auto a = toHip<double>({1, 10, 20, 30}, {4, 1});
  CHECK(eq(am::bc_pow(a, 2.0), {1, 100, 400, 900}));
  auto inv = am::bc_pow(a, -1.0).toCpu();
  auto p2 = am::bc_pow(2.0, a).toCpu();
  const double want_inv[4] = {1.0, 1.0 / 10.0, 1.0 / 20.0, 1.0 / 30.0};
  const double want_p2[4] = {2.0, 1024.0, 1048576.0, 1073741824.0};
  for (int i = 0; i < 4; ++i) {
    CHECK(std::fabs(inv[i] - want_inv[i]) <= 4e-16 * want_inv[i]);
    CHECK(std::fabs(p2[i] - want_p2[i]) <= 4e-16 * want_p2[i]);
  }
  auto b = a.clone();
  b.bc_ipow(2.0);
  CHECK(eq(b, {1, 100, 400, 900}));
  // tests/tensor/test_math_functions.nim:20-45: reciprocal is one IEEE division
  CHECK(eq(am::reciprocal(a), {1.0, 1.0 / 10.0, 1.0 / 20.0, 1.0 / 30.0}));
  // tests/tensor/test_ufunc.nim:31-44: cos and ln against the scalar functions
  auto c = am::cos(toHip<double>({1, 2, 3, 4, 5, 6}, {2, 3})).toCpu();
  auto l = am::ln(toHip<double>({7, 8, 9, 10, 11, 12}, {3, 2})).toCpu();
  for (int i = 0; i < 6; ++i) {
    CHECK(std::fabs(c[i] - std::cos(1.0 + i)) <= 1e-15);
    CHECK(std::fabs(l[i] - std::log(7.0 + i)) <= 1e-15);
  }
  CHECK(eq(am::floor(toHip<float>({-1.5f, -0.5f, 0.5f, 2.0f}, {4})), {-2, -1, 0, 2}));
  CHECK(eq(am::ceil(toHip<float>({-1.5f, -0.5f, 0.5f, 2.0f}, {4})), {-1, -0.0f, 1, 2}));
  CHECK(eq(am::trunc(toHip<float>({-1.5f, -0.5f, 0.5f, 2.0f}, {4})), {-1, -0.0f, 0, 2}));
  CHECK(eq(am::round(toHip<float>({-1.5f, -0.5f, 0.5f, 2.5f}, {4})), {-2, -1, 1, 3}));
  EXPECT_THROW(am::unary(AM_UOP_LN, toHip<int32_t>({1, 2}, {2})), std::invalid_argument);
}

static void argmax_argmin() {
  // tests/tensor/test_aggregate.nim:112-119, 158-166
  auto a = toHip<int32_t>({0, 4, 7, 1, 9, 5, 3, 4, 1}, {3, 3});
  CHECK(eq(am::argmax(a, 0), std::vector<int64_t>{2, 1, 0}));
  CHECK(eq(am::argmax(a, 1), std::vector<int64_t>{2, 1, 1}));
  CHECK(eq(am::argmin(a, 0), std::vector<int64_t>{0, 0, 2}));
  CHECK(eq(am::argmin(a, 1), std::vector<int64_t>{0, 0, 2}));
  auto r = am::argmax_max(toHip<float>({1, 5, 5, 2}, {1, 4}), 1);
  CHECK(eq(r.first, std::vector<int64_t>{1}) && eq(r.second, {5.0f}) && r.first.shape == (Shape{1, 1}));
}

template <typename T> static void conv_literals() {
  // tests/nn_primitives/test_nnp_convolution.nim:21-46 and :54-134: the convolution as one launch (float types) and as
  // im2col + batched GEMM (every type)
  {  // simple_pad1
    auto x = toHip<T>({1, 2, 0, 0, 5, 3, 0, 4, 0, 0, 0, 7, 9, 3, 0, 0}, {1, 1, 4, 4});
    auto k = toHip<T>({1, 1, 1, 1, 1, 0, 1, 0, 0}, {1, 1, 3, 3});
    auto b = toHip<T>(std::vector<T>{0}, {1});   // ({0} alone would be a null pointer)
    const std::vector<T> want = {1, 8, 5, 0, 8, 11, 5, 4, 8, 17, 10, 11, 9, 12, 10, 7};
    CHECK(eq(am::conv2d(x, k, &b, 1, 1, 1, 1), want));
    CHECK(eq(am::conv2d(x, k, &b, 1, 1, 1, 1, false, false), want));   // im2col + batched GEMM
    std::vector<T> clipped = want;
    for (auto& v : clipped) v = v > T(0) ? v : T(0);
    CHECK(eq(am::conv2d(x, k, &b, 1, 1, 1, 1, true), clipped));
  }
  {  // strided_pad1_stride2
    auto x = toHip<T>({2, 2, 0, 2, 1, 0, 1, 1, 0, 2, 1, 2, 1, 2, 1, 2, 2, 0, 0, 2, 2, 1, 1, 1, 2, 2, 0, 1, 1, 1, 2, 2, 0, 0, 2, 2, 2, 1, 0, 0, 1, 1, 2, 2, 0, 2, 1, 1, 1, 0, 0, 1, 2, 2, 0, 1, 1, 1, 1, 0, 2, 1, 2, 2, 0, 0, 2, 2, 2, 1, 0, 0, 2, 2, 1}, {1, 3, 5, 5});
    auto k = toHip<T>({-1, -1, -1, 1, 0, 1, 0, -1, 0, 1, 0, -1, 1, -1, 1, 0, 1, 0, 0, 0, 1, -1, -1, -1, -1, 0, 0, 0, 1, 0, 1, -1, -1, 1, 1, -1, -1, 0, 1, -1, -1, 1, 1, 1, 0, 0, 1, 1, -1, 1, -1, -1, -1, 0}, {2, 3, 3, 3});
    auto b = toHip<T>({1, 0}, {2});
    const std::vector<T> want = {2, -2, 0, -3, 2, -5, -2, -1, 0, -7, 1, 0, 3, -3, 2, 1, 3, -2};
    CHECK(eq(am::conv2d(x, k, &b, 1, 1, 2, 2), want));
    CHECK(eq(am::conv2d(x, k, &b, 1, 1, 2, 2, false, false), want));   // im2col + batched GEMM
    std::vector<T> clipped = want;
    for (auto& v : clipped) v = v > T(0) ? v : T(0);
    CHECK(eq(am::conv2d(x, k, &b, 1, 1, 2, 2, true), clipped));
  }
}

template <typename T> static void conv_backward_known_answer() {
  // conv2d_backward (nnp_convolution.nim:65-107) on a case worked by hand: two copies of the 3 x 3 image 1..9, one
  // 2 x 2 kernel {1, 2, 3, 4}, grad_output all ones. grad_weight[kh, kw] sums the image under each kernel entry,
  // grad_input is the kernel spread over the positions it was applied at, grad_bias counts the outputs.
  auto x = toHip<T>({1, 2, 3, 4, 5, 6, 7, 8, 9, 1, 2, 3, 4, 5, 6, 7, 8, 9}, {2, 1, 3, 3});
  auto k = toHip<T>({1, 2, 3, 4}, {1, 1, 2, 2});
  auto g = toHip<T>({1, 1, 1, 1, 1, 1, 1, 1}, {2, 1, 2, 2});
  auto r = am::conv2d_backward(x, k, true, 0, 0, 1, 1, g);
  CHECK(r.weight.shape == (Shape{1, 1, 2, 2}) && eq(r.weight, {24, 32, 48, 56}));
  CHECK(r.input.shape == (Shape{2, 1, 3, 3}) && eq(r.input, {1, 3, 2, 4, 10, 6, 3, 7, 4, 1, 3, 2, 4, 10, 6, 3, 7, 4}));
  CHECK(r.bias.shape == (Shape{1, 1, 1}) && eq(r.bias, {8}));
  auto nb = am::conv2d_backward(x, k, false, 0, 0, 1, 1, g);
  CHECK(nb.bias.rank() == 0 && eq(nb.weight, {24, 32, 48, 56}));
  // an output row of four pixels (one 16-byte float vector: the weight gradient gathered from the image): the 2 x 5 image
  // 1..10 under a 2 x 2 kernel, grad_output all ones; each entry sums four neighbours of its row
  auto wide = am::conv2d_backward(toHip<T>({1, 2, 3, 4, 5, 6, 7, 8, 9, 10}, {1, 1, 2, 5}), k, false, 0, 0, 1, 1, toHip<T>({1, 1, 1, 1}, {1, 1, 1, 4}));
  CHECK(eq(wide.weight, {10, 14, 30, 34}) && eq(wide.input, {1, 3, 3, 3, 2, 3, 7, 7, 7, 4}));
  // col2im on its own: the column matrix of ones of that geometry counts the patches over each pixel
  auto ones = toHip<T>(std::vector<T>(16, T(1)), {1, 4, 4});
  CHECK(eq(am::col2im(ones, 1, 3, 3, 2, 2), {1, 2, 1, 2, 4, 2, 1, 2, 1}));
  bool threw = false;
  try { am::conv2d_backward(x, k, true, 0, 0, 1, 1, x); } catch (const std::invalid_argument&) { threw = true; }
  CHECK(threw);
}

static void gru_cell_literals() {
  // tests/nn_primitives/test_nnp_gru.nim:10-57: one GRU cell against the values the reference took from PyTorch / cuDNN
  auto x = toHip<double>({0.1, 0.2, 0.3, 0.4, -0.1, -0.2, -0.3, -0.4, 0.5, 0.6, 0.7, 0.8}, {3, 4});
  auto W3 = toHip<double>({0.9, 0.8, 0.7, 0.6, 0.8, 0.7, 0.6, 0.5, 0.7, 0.6, 0.5, 0.4, 0.6, 0.5, 0.4, 0.3, 0.5, 0.4, 0.3, 0.2, 0.4, 0.3, 0.2, 0.1}, {6, 4});
  auto U3 = toHip<double>({-0.3, -0.1, -0.2, 0.0, -0.3, -0.1, -0.2, 0.0, -0.3, -0.1, -0.2, 0.0}, {6, 2});
  auto bW3 = toHip<double>({0.1, 0.2, 0.3, 0.4, 0.5, 0.6}, {1, 6});
  auto bU3 = toHip<double>({-0.1, -0.2, -0.3, -0.4, -0.5, -0.6}, {1, 6});
  const std::vector<double> want = {-0.5317437280, -0.4752916969, -0.3930421219, -0.3209550879, -0.7325259335, -0.6429624731};
  auto close = [&](const am::HipTensor<double>& h) {
    const auto got = h.toCpu();
    double err = 0;
    for (size_t i = 0; i < want.size(); ++i) err += std::fabs(got[i] - want[i]) / std::fabs(want[i]);
    return err / want.size() < 1e-8;
  };
  auto h = toHip<double>({-1, -1, -1, -1, -1, -1}, {3, 2});
  am::gru_cell_inference(x, W3, U3, bW3, bU3, h);
  CHECK(close(h));
  auto h2 = toHip<double>({-1, -1, -1, -1, -1, -1}, {3, 2});
  std::vector<am::HipTensor<double>> saved;
  am::gru_cell_inference(x, W3, U3, bW3, bU3, h2, &saved);
  CHECK(close(h2) && saved.size() == 4 && saved[0].shape == (Shape{3, 2}));
  const auto z = saved[1].toCpu(), n = saved[2].toCpu(), hn = h2.toCpu();
  for (size_t i = 0; i < 6; ++i) CHECK(std::fabs((1 - z[i]) * n[i] + z[i] * -1.0 - hn[i]) < 1e-15);
}

static void sigmoid_loss_and_sgd() {
  // sigmoid cross-entropy at x = 0 is ln 2 per element whatever the target; its gradient there is (0.5 - y) / batch
  auto x = toHip<double>({0, 0, 0, 0, 0, 0}, {2, 3});
  auto y = toHip<double>({1, 0, 0.5, 0, 1, 0.25}, {2, 3});
  CHECK(std::fabs(am::sigmoid_cross_entropy(x, y) - 3 * std::log(2.0)) < 1e-14);
  CHECK(eq(am::sigmoid_cross_entropy_backward(2.0, x, y), {-0.5, 0.5, 0.0, 0.5, -0.5, 0.25}));
  // every parameter updated by one launch: value - lr * gradient
  auto w = toHip<float>({1, 2, 3, 4}, {2, 2});
  auto b = toHip<float>({10, 20, 30}, {3});
  const auto gw = toHip<float>({1, 1, 2, 2}, {2, 2});
  const auto gb = toHip<float>({4, 8, 12}, {3});
  am::sgd_update<float>({&w, &b}, {&gw, &gb}, 0.5f);
  CHECK(eq(w, {0.5f, 1.5f, 2.0f, 3.0f}) && eq(b, {8, 16, 24}));
}

static void graph_with_temporaries() {
  // A sequence with temporaries recorded as it is: out <- relu(a * w + a) through three operator results that are
  // dropped inside the recorded function; replays follow new values written into `a`.
  auto a = toHip<float>({1, -2, 3, -4}, {2, 2});
  auto w = toHip<float>({1, 0, 0, 1}, {2, 2});
  am::HipTensor<float> out(Shape{2, 2});
  auto step = [&]() {
    auto prod = a * w;            // temporary
    auto sum = prod + a;          // temporary
    out.copy_from(am::unary(AM_UOP_RELU, sum));
  };
  auto g = am::Graph::record(step);
  g.launch();
  CHECK(eq(out, {2, 0, 6, 0}));
  a.copy_from(toHip<float>({-1, 2, -3, 4}, {2, 2}));
  g.launch();
  CHECK(eq(out, {0, 4, 0, 8}));
  am::Graph moved = std::move(g);
  CHECK(bool(moved) && !bool(g));
  moved.launch();
  CHECK(eq(out, {0, 4, 0, 8}));
}

static void loss_literals() {
  // tests/nn_primitives/test_nnp_loss.nim:31-44: one row, truth = class 3, loss 0.0709 within 2e-5, dense and sparse
  auto predicted = toHip<double>({-3.44, 1.16, -0.81, 3.91}, {1, 4});
  auto truth = toHip<double>({0, 0, 0, 1}, {1, 4});
  auto sparse_truth = toHip<int64_t>(std::vector<int64_t>{3}, {1});
  const double dense = am::softmax_cross_entropy(predicted, truth), sparse = am::sparse_softmax_cross_entropy(predicted, sparse_truth);
  CHECK(std::fabs(dense - 0.0709) <= 2e-5 && std::fabs(sparse - 0.0709) <= 2e-5);
  // the gradient: softmax - onehot, scaled; its entries sum to zero and only the true class is negative
  auto g = am::softmax_cross_entropy_backward(1.0, predicted, truth).toCpu();
  auto gs = am::sparse_softmax_cross_entropy_backward(1.0, predicted, sparse_truth).toCpu();
  CHECK(std::fabs(g[0] + g[1] + g[2] + g[3]) < 1e-15 && g[3] < 0 && g[0] > 0 && g[1] > 0 && g[2] > 0);
  CHECK(std::fabs(g[3] - (std::exp(-dense) - 1.0)) < 1e-12);   // softmax of the true class is exp(-loss)
  for (int i = 0; i < 4; ++i) CHECK(std::fabs(g[i] - gs[i]) < 1e-15);
}

static void maxpool_backward() {
  // tests/nn_primitives/test_nnp_maxpool.nim:20-45
  auto a = toHip<float>({1, 1, 2, 4, 5, 6, 7, 8, 3, 2, 1, 0, 1, 2, 3, 4}, {1, 1, 4, 4});
  auto p = am::maxpool2d(a, 2, 2, 0, 0, 2, 2);
  CHECK(eq(p.maxpooled, {6, 8, 3, 4}) && eq(p.max_indices, std::vector<int64_t>{5, 7, 8, 15}));
  auto g = am::maxpool2d_backward(a.shape, p.max_indices, p.maxpooled, 2, 2, 0, 0, 2, 2);
  CHECK(eq(g, {0, 0, 0, 0, 0, 6, 0, 8, 3, 0, 0, 0, 0, 0, 0, 4}));
}

static void fused_linear() {
  // nnp_linear.nim:28-29 + relu on small exact values
  auto x = toHip<float>({1, 2, 3, -1, -2, -3}, {2, 3});
  auto w = toHip<float>({1, 0, 0, 0, 1, 0, 1, 1, 1, -1, -1, -1}, {4, 3});
  auto b = toHip<float>({0.5f, -0.5f, 1, 0}, {1, 4});
  CHECK(eq(am::linear(x, w, b), {1.5f, 1.5f, 7, -6, -0.5f, -2.5f, -5, 6}));
  CHECK(eq(am::linear(x, w, b, true), {1.5f, 1.5f, 7, 0, 0, 0, 0, 6}));
  CHECK(eq(am::bias_relu(x, toHip<float>({-2, 0, 2}, {1, 3})), {0, 2, 5, 0, 0, 0}));
  CHECK(eq(am::relu(x), {1, 2, 3, 0, 0, 0}));
  // nnp_linear.nim:39-55 on values small enough to be exact
  auto g = toHip<float>({1, 0, 2, -1, 0, 1, 0, 1}, {2, 4});
  auto grads = am::linear_backward(x, w, g);
  CHECK(eq(grads.input, {4, 3, 3, -1, 0, -1}));
  CHECK(eq(grads.weight, {1, 2, 3, -1, -2, -3, 2, 4, 6, -2, -4, -6}));
  CHECK(grads.bias.shape == (Shape{1, 4}) && eq(grads.bias, {1, 1, 2, 0}));
  // nnp_activation.nim:61-74
  CHECK(eq(am::relu_backward(toHip<float>({1, 2, 3, 4, 5, 6}, {2, 3}), x), {1, 2, 3, 0, 0, 0}));
  CHECK(eq(am::sigmoid_backward(toHip<float>({4, 16}, {2}), toHip<float>({0.5f, 0.25f}, {2})), {1, 3}));
  CHECK(eq(am::tanh_backward(toHip<float>({4, 8}, {2}), toHip<float>({0.5f, -0.5f}, {2})), {3, 6}));
}

template <typename T>
static void aggregates() {
  // tests/tensor/test_aggregate.nim:20-84
  auto t = toHip<T>({0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11}, {4, 3});
  CHECK(am::sum(t) == T(66));
  CHECK(eq(am::sum(t, 0), {18, 22, 26}));
  CHECK(eq(am::sum(t, 1), {3, 12, 21, 30}));
  CHECK(am::sum(t, 0).shape == (am::Shape{1, 3}) && am::sum(t, 1).shape == (am::Shape{4, 1}));
  CHECK(am::product(t) == T(0));
  auto a = toHip<T>({1, 2, 4, 8, 16, 32}, {2, 3});
  CHECK(am::product(a) == T(32768));
  CHECK(eq(am::product(a, 0), {8, 32, 128}));
  CHECK(eq(am::product(a, 1), {8, 4096}));
  auto v = toHip<T>({2, -1, 3, -3, 5, 0}, {6});
  CHECK(am::min(v) == T(-3) && am::max(v) == T(5));
  auto b = toHip<T>({1, 2, 3, -4, 0, 4, -2, 5}, {2, 4});
  CHECK(eq(am::min(b, 0), {0, 2, -2, -4}));
  CHECK(eq(am::min(b, 1), {-4, -2}));
  CHECK(eq(am::max(b, 0), {1, 4, 3, 5}));
  CHECK(eq(am::max(b, 1), {3, 5}));
  CHECK(eq(am::sum(t.transpose(), 0), {3, 12, 21, 30}));
  EXPECT_THROW(am::sum(t, 2), std::out_of_range);
  if (std::is_floating_point<T>::value) {
    CHECK(am::mean(t) == T(5.5));
    CHECK(eq(am::mean(t, 0), {T(4.5), T(5.5), T(6.5)}));
    CHECK(eq(am::mean(t, 1), {1, 4, 7, 10}));
  } else {
    CHECK(am::mean(t) == T(5));
    CHECK(am::mean(toHip<T>({-7, 2, 1}, {3})) == T(-1));
  }
  // tests/nn_primitives/test_nnp_maxpool.nim:20-31
  auto img = toHip<T>({1, 1, 2, 4, 5, 6, 7, 8, 3, 2, 1, 0, 1, 2, 3, 4}, {1, 1, 4, 4});
  auto mp = am::maxpool2d(img, 2, 2, 0, 0, 2, 2);
  CHECK(eq(mp.maxpooled, {6, 8, 3, 4}));
  CHECK(mp.max_indices.toCpu() == (std::vector<int64_t>{5, 7, 8, 15}));
}

static void comparisons_and_predicates() {
  using U8 = std::vector<uint8_t>;
  // tests/tensor/test_higherorder.nim:103-112: a map body with a bool result, one device pass
  auto a = toHip<int64_t>({10, 2, 4, 12}, {4});
  auto b = toHip<int64_t>({4, 4, 4, 4}, {4});
  CHECK(am::map2_bool(AM_CMP_MOD_IS_ZERO, a, b).toCpu() == (U8{0, 0, 1, 1}));
  // tests/tensor/test_operators_comparison.nim:57-79
  auto x = toHip<int32_t>({0, 1, 2, 3}, {4});
  auto y = toHip<int32_t>({0, 2, 1, 3}, {4});
  CHECK(am::bc_eq(x, y).toCpu() == (U8{1, 0, 0, 1}));
  CHECK(am::bc_lt(x, y).toCpu() == (U8{0, 1, 0, 0}));
  CHECK(am::bc_ge(x, 2).toCpu() == (U8{0, 0, 1, 1}));
  CHECK(am::bc_le(2, x).toCpu() == (U8{0, 0, 1, 1}));
  // implicit broadcasting [4,1] vs [1,3]
  auto c = toHip<double>({0, 1, 2, 3}, {4, 1});
  auto d = toHip<double>({0, 1, 2}, {1, 3});
  auto gt = am::bc_gt(c, d);
  CHECK(gt.shape == (Shape{4, 3}) && gt.toCpu() == (U8{0, 0, 0, 1, 0, 0, 1, 1, 0, 1, 1, 1}));
  EXPECT_THROW(am::bc_eq(toHip<double>(std::vector<double>(8, 0), {4, 2}), d), std::invalid_argument);
  // tests/tensor/test_math_functions.nim:115-164
  auto s = toHip<double>({-5.3, 42.0, -0.0, 0.01, 10.7, -0.001, 0.9, -125.3}, {8});
  CHECK(am::sgn(s).toCpu() == (std::vector<int64_t>{-1, 1, 0, 1, 1, -1, 1, -1}));
  const double inf = 1.0 / 0.0, nan = std::nan("");
  auto f = toHip<double>({0.0, -0.0, inf, -inf, nan}, {5});
  CHECK(am::isNaN(f).toCpu() == (U8{0, 0, 0, 0, 1}) && am::isNotNaN(f).toCpu() == (U8{1, 1, 1, 1, 0}));
  CHECK(am::classify(f).toCpu() == (U8{2, 3, 5, 6, 4}));   // fcZero, fcNegZero, fcInf, fcNegInf, fcNan
  // test_math_functions.nim:62-68 clamp / mclamp
  auto k = toHip<int64_t>({-5, 2, 3, 5, 10, 0, 1, -1}, {8});
  CHECK(eq(am::clamp(k, int64_t(-2), int64_t(2)), {-2, 2, 2, 2, 2, 0, 1, -1}));
  k.mclamp(-2, 2);
  CHECK(eq(k, {-2, 2, 2, 2, 2, 0, 1, -1}));
  // :125-130 floorMod on arange(-70.7, 50.0, 34.7), :119-123 copySign
  auto m = toHip<double>({-70.7, -36.0, -1.3, 33.4}, {4});
  const std::vector<double> ts = am::floorMod(m, 3.0).toCpu(), st = am::floorMod(3.0, m).toCpu();
  const double wts[4] = {1.3, -0.0, 1.7, 0.4}, wst[4] = {-67.7, -33.0, -0.9, 3.0};
  for (int i = 0; i < 4; ++i) CHECK(std::fabs(ts[i] - wts[i]) < 1e-9 && std::fabs(st[i] - wst[i]) < 1e-9);
  CHECK(eq(am::copySign(toHip<double>({-5.3, 42.0, 0.9}, {3}), toHip<double>({-4.0, -3.0, 2.0}, {3})), {-5.3, -42.0, 0.9}));
  CHECK(eq(am::degToRad(toHip<double>({180.0, 0.0}, {2})), {3.14159265358979323846, 0.0}));
}

static void display() {
  // tests/tensor/test_display.nim:143-151 (3D table) and :85-92 (single column), on device tensors
  std::vector<int64_t> v(24);
  for (int i = 0; i < 24; ++i) v[i] = i + 1;
  const std::string got = am::pretty(toHip<int64_t>(v, {2, 3, 4}));
  const std::string want =
      "HipTensor[system.int] of shape \"[2, 3, 4]\" on backend \"Hip\"\n"
      "          0                      1           \n"
      "|1      2     3     4| |13    14    15    16|\n"
      "|5      6     7     8| |17    18    19    20|\n"
      "|9     10    11    12| |21    22    23    24|\n";
  CHECK(got == want);
  auto col = toHip<int64_t>({1, 2, 3, 4, 5}, {1, 5}).transpose();   // a strided view: gathered on the device first
  CHECK(am::pretty(col, -1, "||") == "| 1|\n| 2|\n| 3|\n| 4|\n| 5|");
  CHECK(am::pretty(col, -1, "<>") == "HipTensor[int]<5,1>:[[1], [2], [3], [4], [5]]");
  CHECK(am::pretty(am::bc_ge(toHip<float>({0.5f, 2.0f}, {2}), 1.0f), -1, "<>") == "HipTensor[bool]<2>:[false, true]");
  CHECK(am::pretty(toHip<float>({0.9532932f, 0.12945823f}, {2}), 4, "[]") == "[0.9533, 0.1295]");
}

static void softmax_rows() {
  auto x = toHip<double>({1, 2, 3, 1000, 1000, 1000}, {2, 3});
  const std::vector<double> s = am::softmax(x).toCpu();
  const double e1 = std::exp(1.0), e2 = std::exp(2.0), e3 = std::exp(3.0), z = e1 + e2 + e3;
  CHECK(std::fabs(s[0] - e1 / z) < 1e-15 && std::fabs(s[1] - e2 / z) < 1e-15 && std::fabs(s[2] - e3 / z) < 1e-15);
  CHECK(std::fabs(s[3] - 1.0 / 3) < 1e-15 && std::fabs(s[4] - 1.0 / 3) < 1e-15 && std::fabs(s[5] - 1.0 / 3) < 1e-15);
}

// tests/io/test_numpy.nim:15-96 on the data files of the reference's own test
static void npy_files(const std::string& dir) {
  const std::vector<int64_t> e1 = {1, 2, 3, 4}, e2 = {1, 2, 3, 4, 5, 6, 7, 8};
  for (const char* stem : {"int", "f32LE", "u64BE"}) {
    const std::string s = dir + "/" + stem;
    CHECK(am::read_npy<int64_t>(s + ".npy").toCpu() == e1);
    auto c = am::read_npy<int64_t>(s + "_2D_c.npy"), f = am::read_npy<int64_t>(s + "_2D_f.npy");
    CHECK(c.shape == (am::Shape{2, 4}) && c.toCpu() == e2 && c.is_C_contiguous());
    CHECK(f.shape == (am::Shape{2, 4}) && f.toCpu() == e2 && f.is_F_contiguous() && !f.is_C_contiguous());
    CHECK(eq(am::read_npy<float>(s + "_2D_f.npy"), {1, 2, 3, 4, 5, 6, 7, 8}));
  }
  auto same = [](const std::string& a, const std::string& b) {
    std::ifstream fa(a, std::ios::binary), fb(b, std::ios::binary);
    const std::string ca((std::istreambuf_iterator<char>(fa)), std::istreambuf_iterator<char>());
    const std::string cb((std::istreambuf_iterator<char>(fb)), std::istreambuf_iterator<char>());
    return !ca.empty() && ca == cb;
  };
  const std::string out = "/tmp/am_hip_test_write.npy";
  am::write_npy(toHip<int64_t>({1, 2, 3, 4}, {4}), out);
  CHECK(same(out, dir + "/int.npy"));
  auto t2 = toHip<int64_t>({1, 2, 3, 4, 5, 6, 7, 8}, {2, 4});
  am::write_npy(t2, out);
  CHECK(same(out, dir + "/int_2D_c.npy"));
  am::write_npy(toHip<int64_t>({1, 5, 2, 6, 3, 7, 4, 8}, {4, 2}).transpose(), out);   // column-major [2, 4]
  CHECK(same(out, dir + "/int_2D_f.npy"));
  am::write_npy(toHip<float>({1, 2, 3, 4, 5, 6, 7, 8}, {2, 4}), out);
  CHECK(same(out, dir + "/f32LE_2D_c.npy"));
  am::write_npy(toHip<float>({1, 5, 2, 6, 3, 7, 4, 8}, {4, 2}).transpose(), out);
  CHECK(same(out, dir + "/f32LE_2D_f.npy"));
  EXPECT_THROW(am::read_npy<float>(dir + "/does_not_exist.npy"), std::ios_base::failure);
  std::remove(out.c_str());
}

int main(int argc, char** argv) {
  try {
    gemm_literals<float>();
    gemm_literals<double>();
    gemm_literals<int32_t>();
    gemm_literals<int64_t>();
    integer_slices();
    add_sub_scalars();
    unsigned_ring_ops<uint32_t>();
    unsigned_ring_ops<uint64_t>();
    scalar_broadcast();
    broadcasting<float>();
    broadcasting<double>();
    broadcasting<int32_t>();
    broadcasting<int64_t>();
    fused_linear();
    variance_std();
    pow_and_universal_functions();
    argmax_argmin();
    conv_literals<float>();
  conv_literals<double>();
  conv_literals<int32_t>();
  conv_literals<int64_t>();
  loss_literals();
  graph_with_temporaries();
  sigmoid_loss_and_sgd();
  gru_cell_literals();
  conv_backward_known_answer<float>();
  conv_backward_known_answer<double>();
  conv_backward_known_answer<int32_t>();
  conv_backward_known_answer<int64_t>();
  maxpool_backward();
    aggregates<float>();
    aggregates<double>();
    aggregates<int32_t>();
    aggregates<int64_t>();
    softmax_rows();
    comparisons_and_predicates();
    display();
    if (argc > 1) npy_files(argv[1]);
    am::sync();
  } catch (const std::exception& e) {
    std::printf("unexpected exception: %s\n", e.what());
    return 2;
  }
  std::printf("%d checks, %d failed\n", g_checked, g_failed);
  return g_failed ? 1 : 0;
}
