// Weight repacking for the GEMMs that read their operands in tile order (kernels: gemm_fp6.h, gemm_tile8.h;
// operand formats: fp6_format.h; the activation side is produced by the quantize kernel).
#include "gemm_fp6.h"

namespace quik {
namespace {

constexpr int kThreads = 256;

// 8 nibbles of a packed int4 dword (two's complement codes) -> two dwords of level bytes
__device__ __forceinline__ void nibbles_to_level_bytes(uint32_t w, uint32_t &lo, uint32_t &hi) {
  w ^= 0x88888888u;  // code + 8
  // element 2i is the low nibble of byte i: bytes (e0 e1 e2 e3) come from nibbles 0..3 = bytes 0, 1 of w
  const uint32_t even = w & 0x0F0F0F0Fu, odd = (w >> 4) & 0x0F0F0F0Fu;   // e0 e2 e4 e6 / e1 e3 e5 e7
  lo = __builtin_amdgcn_perm(odd, even, 0x05010400u);   // e0 e1 e2 e3
  hi = __builtin_amdgcn_perm(odd, even, 0x07030602u);   // e4 e5 e6 e7
}

// weights [N, K/2] packed int4 and outlier weights [N, F] (16-bit patterns) -> operand buffer; one
// workgroup per row, one lane per fragment / 16-byte outlier chunk
__global__ __launch_bounds__(kThreads) void pack_weight_kernel(const uint8_t *__restrict__ qw,
                                                               const uint16_t *__restrict__ fp_w, int64_t rows,
                                                               int64_t K, int64_t F, uint8_t *__restrict__ out) {
  const Fp6Layout l = fp6_layout(rows, K, F);
  const int64_t frags_per_row = l.steps * 2;
  const int64_t row = blockIdx.x;
  for (int64_t c = threadIdx.x; c < F / 8; c += kThreads)
    *reinterpret_cast<uint4 *>(out + fp6_outlier_offset(l, row, c >> 1, static_cast<int>(c & 1))) =
        *reinterpret_cast<const uint4 *>(fp_w + row * F + c * 8);
  __shared__ int total;
  if (threadIdx.x == 0) total = 0;
  __syncthreads();
  int sum = 0;
  for (int64_t f = threadIdx.x; f < frags_per_row; f += kThreads) {
    const uint4 v = *reinterpret_cast<const uint4 *>(qw + row * (K / 2) + f * 16);  // 32 nibbles
    uint32_t b[8];
    nibbles_to_level_bytes(v.x, b[0], b[1]);
    nibbles_to_level_bytes(v.y, b[2], b[3]);
    nibbles_to_level_bytes(v.z, b[4], b[5]);
    nibbles_to_level_bytes(v.w, b[6], b[7]);
#pragma unroll
    for (int i = 0; i < 8; ++i) sum = __builtin_amdgcn_udot4(b[i], 0x01010101u, sum, false);
    uint32_t o[6];
    fp6_pack_fragment(b, o);
    fp6_store_fragment(out, l, row, f, o);
  }
  atomicAdd(&total, sum);
  __syncthreads();
  if (threadIdx.x == 0) reinterpret_cast<int32_t *>(out + l.sums_off)[row] = total;
}

// int8 weights [N, K] and outlier weights [N, F] -> int8 operand buffer in tile order; one lane per 16-byte chunk
__global__ __launch_bounds__(kThreads) void pack_weight8_kernel(const uint8_t *__restrict__ qw,
                                                                const uint16_t *__restrict__ fp_w, int64_t rows,
                                                                int64_t K, int64_t F, uint8_t *__restrict__ out) {
  const Tile8Layout l = tile8_layout(rows, K, F);
  const int64_t row = blockIdx.x;
  for (int64_t c = threadIdx.x; c < K / 16; c += kThreads)
    *reinterpret_cast<uint4 *>(out + tile8_offset(l, row, c >> 1, static_cast<int>(c & 1))) =
        *reinterpret_cast<const uint4 *>(qw + row * K + c * 16);
  for (int64_t c = threadIdx.x; c < F / 8; c += kThreads)
    *reinterpret_cast<uint4 *>(out + tile8_offset(l, row, l.steps + (c >> 1), static_cast<int>(c & 1))) =
        *reinterpret_cast<const uint4 *>(fp_w + row * F + c * 8);
}

}  // namespace
}  // namespace quik

using namespace quik;

extern "C" int64_t quik_tile8_operand_bytes(int64_t rows, int64_t K, int64_t F) {
  if (rows <= 0 || K <= 0 || K % 64 != 0 || F < 0 || F % 32 != 0) return 0;
  return tile8_layout(rows, K, F).bytes;
}

extern "C" int quik_tile8_pack_weight(const int8_t *qw, const void *fp_w, int64_t N, int64_t K, int64_t F, void *out,
                                      void *stream) {
  if (N <= 0 || K <= 0 || F < 0) return QUIK_ERR_SHAPE;
  if (K % 64 != 0 || F % 32 != 0) return QUIK_ERR_ALIGN;
  if (!qw || !out || (F > 0 && !fp_w)) return QUIK_ERR_NULL;
  if (reinterpret_cast<uintptr_t>(qw) % 16 != 0 || reinterpret_cast<uintptr_t>(out) % 256 != 0 ||
      reinterpret_cast<uintptr_t>(fp_w) % 16 != 0)
    return QUIK_ERR_ALIGN;
  if (N > (1 << 30)) return QUIK_ERR_RANGE;
  hipLaunchKernelGGL(pack_weight8_kernel, dim3(static_cast<unsigned>(N)), dim3(kThreads), 0, as_stream(stream),
                     reinterpret_cast<const uint8_t *>(qw), static_cast<const uint16_t *>(fp_w), N, K, F,
                     static_cast<uint8_t *>(out));
  return check_launch();
}

extern "C" int64_t quik_fp6_operand_bytes(int64_t rows, int64_t K, int64_t F) {
  if (rows <= 0 || K <= 0 || K % 128 != 0 || K > 74496 || F < 0 || F % 32 != 0) return 0;
  return fp6_layout(rows, K, F).bytes;
}

extern "C" int quik_fp6_pack_weight(const uint8_t *qw, const void *fp_w, int64_t N, int64_t K, int64_t F, void *out,
                                    void *stream) {
  if (N <= 0 || K <= 0 || F < 0) return QUIK_ERR_SHAPE;
  if (K % 128 != 0 || F % 32 != 0) return QUIK_ERR_ALIGN;
  if (!qw || !out || (F > 0 && !fp_w)) return QUIK_ERR_NULL;
  if (reinterpret_cast<uintptr_t>(qw) % 16 != 0 || reinterpret_cast<uintptr_t>(out) % 256 != 0 ||
      reinterpret_cast<uintptr_t>(fp_w) % 16 != 0)
    return QUIK_ERR_ALIGN;
  if (N > (1 << 30) || K > 74496) return QUIK_ERR_RANGE;
  hipLaunchKernelGGL(pack_weight_kernel, dim3(static_cast<unsigned>(N)), dim3(kThreads), 0, as_stream(stream), qw,
                     static_cast<const uint16_t *>(fp_w), N, K, F, static_cast<uint8_t *>(out));
  return check_launch();
}
