// Stand-alone dequantize kernels (the unfused ops of the reference API) for gfx950.
//
// asymmetric (reference: src/asymmetric/asymmetric.cu:119-173), fp32, this association order:
//   out = storage( f32(acc) * (s_row * s_col) + ((zero + shift * s_row) * w_red + f32(y)) )
// symmetric (reference: src/symmetric/symmetric.cu:91-113), a chain of fp16 roundings:
//   out = fp16( f32( fp16( fp16( fp16(x) * s_row ) * s_col ) ) + f32(y) )
// Both are pure streaming kernels: 16-byte loads and stores, eight outputs per lane.
// This file is compiled with -ffp-contract=off so the products and sums round separately.
#include "common.h"

namespace quik {
namespace {

constexpr int kThreads = 256;

template <bool BF16>
__device__ __forceinline__ float asym_one(int32_t acc, float s, float z, float c, float w, float y, float shift) {
  float t = static_cast<float>(acc);
  const float sh = (z + shift * s) * w;
  t *= s * c;
  t += sh + y;
  return t;
}

template <bool BF16>
__global__ __launch_bounds__(kThreads) void asym_dequant_vec_kernel(
    const int32_t *__restrict__ acc, const uint16_t *__restrict__ meta, const uint16_t *__restrict__ scol,
    const uint16_t *__restrict__ wred, const uint16_t *__restrict__ y, int64_t rows, int64_t cols, float shift,
    uint16_t *__restrict__ out) {
  const int64_t cvecs = cols >> 3;
  const int64_t total = rows * cvecs;
  for (int64_t i = blockIdx.x * int64_t(kThreads) + threadIdx.x; i < total; i += int64_t(gridDim.x) * kThreads) {
    const int64_t r = i / cvecs, cv = i - r * cvecs;
    const int64_t base = r * cols + cv * 8;
    const uint32_t m = *reinterpret_cast<const uint32_t *>(meta + 2 * r);
    const float s = to_f32<BF16>(static_cast<uint16_t>(m & 0xFFFFu));
    const float z = to_f32<BF16>(static_cast<uint16_t>(m >> 16));
    const int4 a0 = *reinterpret_cast<const int4 *>(acc + base);
    const int4 a1 = *reinterpret_cast<const int4 *>(acc + base + 4);
    const uint4 yv = *reinterpret_cast<const uint4 *>(y + base);
    const uint4 cvv = *reinterpret_cast<const uint4 *>(scol + cv * 8);
    const uint4 wv = *reinterpret_cast<const uint4 *>(wred + cv * 8);
    const int32_t a[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
    const uint32_t yw[4] = {yv.x, yv.y, yv.z, yv.w};
    const uint32_t cw[4] = {cvv.x, cvv.y, cvv.z, cvv.w};
    const uint32_t ww[4] = {wv.x, wv.y, wv.z, wv.w};
    uint32_t o[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float r0 = asym_one<BF16>(a[2 * k], s, z, to_f32<BF16>(cw[k] & 0xFFFFu), to_f32<BF16>(ww[k] & 0xFFFFu),
                                      to_f32<BF16>(yw[k] & 0xFFFFu), shift);
      const float r1 = asym_one<BF16>(a[2 * k + 1], s, z, to_f32<BF16>(cw[k] >> 16), to_f32<BF16>(ww[k] >> 16),
                                      to_f32<BF16>(yw[k] >> 16), shift);
      o[k] = static_cast<uint32_t>(from_f32<BF16>(r0)) | (static_cast<uint32_t>(from_f32<BF16>(r1)) << 16);
    }
    *reinterpret_cast<uint4 *>(out + base) = make_uint4(o[0], o[1], o[2], o[3]);
  }
}

template <bool BF16>
__global__ __launch_bounds__(kThreads) void asym_dequant_scalar_kernel(
    const int32_t *__restrict__ acc, const uint16_t *__restrict__ meta, const uint16_t *__restrict__ scol,
    const uint16_t *__restrict__ wred, const uint16_t *__restrict__ y, int64_t rows, int64_t cols, float shift,
    uint16_t *__restrict__ out) {
  const int64_t total = rows * cols;
  for (int64_t i = blockIdx.x * int64_t(kThreads) + threadIdx.x; i < total; i += int64_t(gridDim.x) * kThreads) {
    const int64_t r = i / cols, c = i - r * cols;
    const float v = asym_one<BF16>(acc[i], to_f32<BF16>(meta[2 * r]), to_f32<BF16>(meta[2 * r + 1]),
                                   to_f32<BF16>(scol[c]), to_f32<BF16>(wred[c]), to_f32<BF16>(y[i]), shift);
    out[i] = from_f32<BF16>(v);
  }
}

template <typename T>
__device__ __forceinline__ _Float16 sym_to_half(T v) {
  return static_cast<_Float16>(static_cast<float>(static_cast<int>(v)));  // exact below 2^24, inf above 65519
}
template <>
__device__ __forceinline__ _Float16 sym_to_half<uint16_t>(uint16_t v) {
  return __builtin_bit_cast(_Float16, v);
}

template <typename T>
__global__ __launch_bounds__(kThreads) void sym_dequant_kernel(const T *__restrict__ x,
                                                               const uint16_t *__restrict__ srow,
                                                               const uint16_t *__restrict__ scol,
                                                               const uint16_t *__restrict__ y, int64_t rows,
                                                               int64_t cols, uint16_t *__restrict__ out) {
  const int64_t total = rows * cols;
  for (int64_t i = blockIdx.x * int64_t(kThreads) + threadIdx.x; i < total; i += int64_t(gridDim.x) * kThreads) {
    const int64_t r = i / cols, c = i - r * cols;
    _Float16 t = sym_to_half<T>(x[i]);
    t = t * __builtin_bit_cast(_Float16, srow[r]);
    t = t * __builtin_bit_cast(_Float16, scol[c]);
    const float sum = static_cast<float>(t) + to_f32<false>(y[i]);
    out[i] = from_f32<false>(sum);
  }
}

// Epilogue of the reference's asymmetric fused GEMM, fp16 arithmetic with one rounding per operation
// (reference: include/asymmetric/epilogue/thread/linear_combination_dequant.h:155-162):
//   ((h(acc) * scale_col) * scale_row + (zero_row + h(shift) * scale_row) * w_reduced) + y
__global__ __launch_bounds__(kThreads) void asym_fused_chain_kernel(
    const int32_t *__restrict__ acc, const uint16_t *__restrict__ srow, const uint16_t *__restrict__ scol,
    _Float16 shift, const uint16_t *__restrict__ zrow, const uint16_t *__restrict__ wred,
    const uint16_t *__restrict__ y, int64_t rows, int64_t cols, uint16_t *__restrict__ out) {
  const int64_t total = rows * cols;
  for (int64_t i = blockIdx.x * int64_t(kThreads) + threadIdx.x; i < total; i += int64_t(gridDim.x) * kThreads) {
    const int64_t r = i / cols, c = i - r * cols;
    const _Float16 sr = __builtin_bit_cast(_Float16, srow[r]);
    _Float16 t = sym_to_half<int32_t>(acc[i]);
    t = t * __builtin_bit_cast(_Float16, scol[c]);
    t = t * sr;
    _Float16 u = shift * sr;
    u = __builtin_bit_cast(_Float16, zrow[r]) + u;
    u = u * __builtin_bit_cast(_Float16, wred[c]);
    t = t + u;
    t = t + __builtin_bit_cast(_Float16, y[i]);
    out[i] = __builtin_bit_cast(uint16_t, t);
  }
}

int grid_for(int64_t items) {
  int64_t g = (items + kThreads - 1) / kThreads;
  if (g < 1) g = 1;
  if (g > 256 * 64) g = 256 * 64;
  return static_cast<int>(g);
}

}  // namespace
}  // namespace quik

using namespace quik;

extern "C" int quik_asym_dequantize(const int32_t *acc, const void *meta, const void *scale_col,
                                    const void *w_reduced, const void *y, int dtype, int64_t rows, int64_t cols,
                                    int bits, void *out, void *stream) {
  if (bits != 4 && bits != 8) return QUIK_ERR_BITS;
  if (dtype != QUIK_F16 && dtype != QUIK_BF16) return QUIK_ERR_DTYPE;
  if (rows < 0 || cols < 0) return QUIK_ERR_SHAPE;
  if (rows == 0 || cols == 0) return QUIK_OK;
  if (!acc || !meta || !scale_col || !w_reduced || !y || !out) return QUIK_ERR_NULL;
  const float shift = bits == 4 ? 8.0f : 128.0f;
  hipStream_t st = as_stream(stream);
  const uint16_t *m = static_cast<const uint16_t *>(meta), *c = static_cast<const uint16_t *>(scale_col),
                 *w = static_cast<const uint16_t *>(w_reduced), *yy = static_cast<const uint16_t *>(y);
  uint16_t *o = static_cast<uint16_t *>(out);
  auto aligned = [](const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const bool vec = cols % 8 == 0 && aligned(acc) && aligned(c) && aligned(w) && aligned(yy) && aligned(o) &&
                   reinterpret_cast<uintptr_t>(m) % 4 == 0;
  if (vec) {
    const int grid = grid_for(rows * (cols / 8));
    if (dtype == QUIK_F16)
      hipLaunchKernelGGL(asym_dequant_vec_kernel<false>, dim3(grid), dim3(kThreads), 0, st, acc, m, c, w, yy, rows,
                         cols, shift, o);
    else
      hipLaunchKernelGGL(asym_dequant_vec_kernel<true>, dim3(grid), dim3(kThreads), 0, st, acc, m, c, w, yy, rows,
                         cols, shift, o);
  } else {
    const int grid = grid_for(rows * cols);
    if (dtype == QUIK_F16)
      hipLaunchKernelGGL(asym_dequant_scalar_kernel<false>, dim3(grid), dim3(kThreads), 0, st, acc, m, c, w, yy,
                         rows, cols, shift, o);
    else
      hipLaunchKernelGGL(asym_dequant_scalar_kernel<true>, dim3(grid), dim3(kThreads), 0, st, acc, m, c, w, yy, rows,
                         cols, shift, o);
  }
  return check_launch();
}

extern "C" int quik_sym_dequantize(const void *x, int x_bits, const void *scale_row, const void *scale_col,
                                   const void *y, int64_t rows, int64_t cols, void *out, void *stream) {
  if (x_bits != 8 && x_bits != 16 && x_bits != 32) return QUIK_ERR_BITS;
  if (rows < 0 || cols < 0) return QUIK_ERR_SHAPE;
  if (rows == 0 || cols == 0) return QUIK_OK;
  if (!x || !scale_row || !scale_col || !y || !out) return QUIK_ERR_NULL;
  hipStream_t st = as_stream(stream);
  const uint16_t *sr = static_cast<const uint16_t *>(scale_row), *sc = static_cast<const uint16_t *>(scale_col),
                 *yy = static_cast<const uint16_t *>(y);
  uint16_t *o = static_cast<uint16_t *>(out);
  const int grid = grid_for(rows * cols);
  if (x_bits == 8)
    hipLaunchKernelGGL(sym_dequant_kernel<int8_t>, dim3(grid), dim3(kThreads), 0, st, static_cast<const int8_t *>(x),
                       sr, sc, yy, rows, cols, o);
  else if (x_bits == 16)
    hipLaunchKernelGGL(sym_dequant_kernel<uint16_t>, dim3(grid), dim3(kThreads), 0, st,
                       static_cast<const uint16_t *>(x), sr, sc, yy, rows, cols, o);
  else
    hipLaunchKernelGGL(sym_dequant_kernel<int32_t>, dim3(grid), dim3(kThreads), 0, st,
                       static_cast<const int32_t *>(x), sr, sc, yy, rows, cols, o);
  return check_launch();
}

// The reference's fused GEMM + dequantize ops as two launches: the exact int32 product into the
// caller's workspace, then the fp16-arithmetic epilogue of the reference on top of it.
static int int_matmul(const void *A, const void *B, int32_t *acc, int64_t M, int64_t N, int64_t K, int bits,
                      void *stream) {
  if (bits == 4)
    return quik_int4_matmul(static_cast<const uint8_t *>(A), static_cast<const uint8_t *>(B), acc, M, N, K, stream);
  if (bits == 8)
    return quik_int8_matmul(static_cast<const int8_t *>(A), static_cast<const int8_t *>(B), acc, M, N, K, stream);
  return QUIK_ERR_BITS;
}

extern "C" int quik_asym_fused_dequantize(const void *A, const void *B, const void *scale_row, const void *scale_col,
                                          float shift_value, const void *zero_row, const void *w_reduced,
                                          const void *y, int64_t M, int64_t N, int64_t K, int bits,
                                          int32_t *acc_workspace, void *out, void *stream) {
  if (bits != 4 && bits != 8) return QUIK_ERR_BITS;
  if (M < 0 || N < 0 || K <= 0) return QUIK_ERR_SHAPE;
  if (M == 0 || N == 0) return QUIK_OK;
  if (!scale_row || !scale_col || !zero_row || !w_reduced || !y || !out) return QUIK_ERR_NULL;
  const _Float16 shift = static_cast<_Float16>(shift_value);
  const int rc = int_gemm_chain(A, B, scale_row, scale_col, zero_row, w_reduced, __builtin_bit_cast(uint16_t, shift), y,
                                M, N, K, bits, out, as_stream(stream));
  if (rc != kChainNotHandled) return rc;
  // at most 32 rows: product by the weight-streaming kernel into the workspace, epilogue as a second launch
  if (!acc_workspace) return QUIK_ERR_NULL;
  if (int rc2 = int_matmul(A, B, acc_workspace, M, N, K, bits, stream)) return rc2;
  hipLaunchKernelGGL(asym_fused_chain_kernel, dim3(grid_for(M * N)), dim3(kThreads), 0, as_stream(stream),
                     acc_workspace, static_cast<const uint16_t *>(scale_row), static_cast<const uint16_t *>(scale_col),
                     shift, static_cast<const uint16_t *>(zero_row), static_cast<const uint16_t *>(w_reduced),
                     static_cast<const uint16_t *>(y), M, N, static_cast<uint16_t *>(out));
  return check_launch();
}

extern "C" int quik_sym_fused_dequantize(const void *A, const void *B, const void *scale_row, const void *scale_col,
                                         const void *y, int64_t M, int64_t N, int64_t K, int bits,
                                         int32_t *acc_workspace, void *out, void *stream) {
  if (bits != 4 && bits != 8) return QUIK_ERR_BITS;
  if (M < 0 || N < 0 || K <= 0) return QUIK_ERR_SHAPE;
  if (M == 0 || N == 0) return QUIK_OK;
  if (!scale_row || !scale_col || !y || !out) return QUIK_ERR_NULL;
  const int rc = int_gemm_chain(A, B, scale_row, scale_col, nullptr, nullptr, 0, y, M, N, K, bits, out,
                                as_stream(stream));
  if (rc != kChainNotHandled) return rc;
  if (!acc_workspace) return QUIK_ERR_NULL;
  if (int rc2 = int_matmul(A, B, acc_workspace, M, N, K, bits, stream)) return rc2;
  return quik_sym_dequantize(acc_workspace, 32, scale_row, scale_col, y, M, N, out, stream);
}

/* bytes of the int32 workspace the fused dequantize entry points need for this shape (0: none, one launch) */
extern "C" int64_t quik_fused_dequantize_workspace_bytes(int64_t M, int64_t N) {
  return (M > 0 && M <= 32 && N > 0) ? M * N * 4 : 0;
}
