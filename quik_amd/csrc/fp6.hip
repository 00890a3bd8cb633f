// Weight repacking for the GEMMs that read their operands in tile order (kernels: gemm_fp6.h, gemm_tile8.h;
// operand formats: fp6_format.h; the activation side is produced by the quantize kernel).
#include "colmap.h"
#include "gemm_fp6.h"

namespace quik {
namespace {

constexpr int kThreads = 256;

// weights [N, K/2] packed int4 (columns in ascending int_indices order) and outlier weights [N, F] (16-bit
// patterns) -> operand buffer; one workgroup per row, one lane per fragment / 16-byte outlier chunk.
// Position k of the operand takes weight column kperm[k] (the in-place order of the column map, which the
// quantize kernel writes the activation in); the row is staged in LDS and gathered nibble by nibble.
__global__ __launch_bounds__(kThreads) void pack_weight_kernel(const uint8_t *__restrict__ qw,
                                                               const uint16_t *__restrict__ fp_w,
                                                               const uint16_t *__restrict__ kperm,
                                                               const uint32_t *__restrict__ flags, int64_t rows,
                                                               int64_t K, int64_t F, uint8_t *__restrict__ out) {
  extern __shared__ __align__(16) uint8_t row_s[];  // K / 2 bytes
  if (!(flags[0] & 2u)) return;  // the column map has no in-place order (the host refuses such a map first)
  const Fp6Layout l = fp6_layout(rows, K, F);
  const int64_t frags_per_row = l.steps * 2;
  const int64_t row = blockIdx.x;
  for (int64_t c = threadIdx.x; c < F / 8; c += kThreads)
    *reinterpret_cast<uint4 *>(out + fp6_outlier_offset(l, row, c >> 1, static_cast<int>(c & 1))) =
        *reinterpret_cast<const uint4 *>(fp_w + row * F + c * 8);
  for (int64_t c = threadIdx.x; c < K / 32; c += kThreads)
    reinterpret_cast<uint4 *>(row_s)[c] = *reinterpret_cast<const uint4 *>(qw + row * (K / 2) + c * 16);
  __shared__ int total;
  if (threadIdx.x == 0) total = 0;
  __syncthreads();
  int sum = 0;
  for (int64_t f = threadIdx.x; f < frags_per_row; f += kThreads) {
    uint32_t b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint2 kp = *reinterpret_cast<const uint2 *>(kperm + f * 32 + i * 4);  // four positions
      const uint32_t k[4] = {kp.x & 0xFFFFu, kp.x >> 16, kp.y & 0xFFFFu, kp.y >> 16};
      uint32_t w = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t nib = (row_s[k[e] >> 1] >> ((k[e] & 1u) * 4u)) & 0xFu;  // two's complement code
        w |= (nib ^ 8u) << (8 * e);                                              // level = code + 8
      }
      b[i] = w;
      sum = __builtin_amdgcn_udot4(w, 0x01010101u, sum, false);
    }
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

extern "C" int quik_fp6_pack_weight(const uint8_t *qw, const void *fp_w, int64_t N, int64_t K, int64_t F,
                                    const void *colmap, void *out, void *stream) {
  if (N <= 0 || K <= 0 || F < 0) return QUIK_ERR_SHAPE;
  if (K % 128 != 0 || F % 32 != 0) return QUIK_ERR_ALIGN;
  if (!qw || !out || !colmap || (F > 0 && !fp_w)) return QUIK_ERR_NULL;
  if (reinterpret_cast<uintptr_t>(qw) % 16 != 0 || reinterpret_cast<uintptr_t>(out) % 256 != 0 ||
      reinterpret_cast<uintptr_t>(fp_w) % 16 != 0 || reinterpret_cast<uintptr_t>(colmap) % 16 != 0)
    return QUIK_ERR_ALIGN;
  if (N > (1 << 30) || K > 74496 || K + F > kStreamMaxCols) return QUIK_ERR_RANGE;
  if (int rc = colmap_require(colmap, K + F, K, F, as_stream(stream), kColmapStreams | kColmapInPlace)) return rc;
  const ColmapLayout cl = colmap_layout(K + F, K, F);
  const uint8_t *cm = static_cast<const uint8_t *>(colmap);
  hipLaunchKernelGGL(pack_weight_kernel, dim3(static_cast<unsigned>(N)), dim3(kThreads), static_cast<size_t>(K / 2),
                     as_stream(stream), qw, static_cast<const uint16_t *>(fp_w),
                     reinterpret_cast<const uint16_t *>(cm + cl.off_kperm),
                     reinterpret_cast<const uint32_t *>(cm + cl.off_flags), N, K, F, static_cast<uint8_t *>(out));
  return check_launch();
}
