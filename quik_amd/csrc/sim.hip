// The reference's simulated ("fake-quant") activation path on the GPU: per-token asymmetric quantize-dequantize
// of the non-outlier columns, outlier columns passed through (reference: experiments/quant_sim.py,
// asymmetric_quantize :5-7, ActQuantizer.find_params :167-188, ActQuantWrapper.forward :227-256):
//   xmin = min(min_k x, 0), xmax = max(max_k x, 0) over the quantized columns, both zero -> (-1, +1)
//   scale = (xmax - xmin) / maxq;  zero = round(-xmin / scale)
//   out   = scale * (clamp(round(x / scale) + zero, 0, maxq) - zero)      quantized columns
//   out   = x                                                             outlier columns
// fp32 arithmetic on fp16 / bf16 storage, one rounding to the storage type at the end, every operation an IEEE
// one (this file is compiled without contraction; round = round-half-to-even as torch.round), so the result
// equals the same expression evaluated by torch in fp32.  A different zero-point convention from the kernel
// path (MixedQLinear): the two agree to quantisation noise, not bit for bit.
//
// HBM-bound streaming kernel: one 256-thread workgroup per row, the row is read twice (the second read comes from
// L2) and written once; 16-byte accesses, one outlier mask byte per group of 8 columns.
#include "common.h"

namespace quik {
namespace {

constexpr int kThreads = 256;

template <bool BF16>
__global__ __launch_bounds__(kThreads) void act_fake_quant_kernel(const uint16_t *__restrict__ x, int64_t rows,
                                                                  int64_t cols, const uint32_t *__restrict__ mask,
                                                                  float maxq, uint16_t *__restrict__ out, int vec) {
  __shared__ float red[8];
  const int tid = threadIdx.x;
  const float inf = __builtin_inff();
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const uint16_t *xr = x + row * cols;
    uint16_t *orow = out + row * cols;
    float mn = inf, mx = -inf;
    if (vec) {
      for (int64_t g = tid; g < (cols >> 3); g += kThreads) {
        const uint4 v = *reinterpret_cast<const uint4 *>(xr + g * 8);
        const uint32_t mb = (mask[g >> 2] >> ((g & 3) * 8)) & 0xFFu;
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float f = to_f32<BF16>(static_cast<uint16_t>(w[e >> 1] >> (16 * (e & 1))));
          const bool outl = (mb >> e) & 1u;
          mn = fminf(mn, outl ? inf : f);
          mx = fmaxf(mx, outl ? -inf : f);
        }
      }
    } else {
      for (int64_t c = tid; c < cols; c += kThreads) {
        if (!((mask[c >> 5] >> (c & 31)) & 1u)) {
          const float f = to_f32<BF16>(xr[c]);
          mn = fminf(mn, f);
          mx = fmaxf(mx, f);
        }
      }
    }
    mn = wave_min(mn);
    mx = wave_max(mx);
    __syncthreads();  // the previous row's reads of `red` are done
    if ((tid & 63) == 0) {
      red[tid >> 6] = mn;
      red[4 + (tid >> 6)] = mx;
    }
    __syncthreads();
    mn = fminf(fminf(red[0], red[1]), fminf(red[2], red[3]));
    mx = fmaxf(fmaxf(red[4], red[5]), fmaxf(red[6], red[7]));
    float xmin = fminf(mn, 0.0f), xmax = fmaxf(mx, 0.0f);
    if (xmin == 0.0f && xmax == 0.0f) {
      xmin = -1.0f;
      xmax = 1.0f;
    }
    const float scale = (xmax - xmin) / maxq;
    const float zero = __builtin_rintf(-xmin / scale);
    auto fake = [&](uint16_t xb) -> uint16_t {
      const float q = fminf(fmaxf(__builtin_rintf(to_f32<BF16>(xb) / scale) + zero, 0.0f), maxq);
      float r = scale * (q - zero);
      // the product is an fp32 value of its own: without this the compiler merges the multiply and the conversion
      // into one mixed-precision instruction that rounds once, straight to fp16, and one result in a few million
      // then differs from the fp32 expression rounded afterwards
      asm volatile("" : "+v"(r));
      return from_f32<BF16>(r);
    };
    if (vec) {
      for (int64_t g = tid; g < (cols >> 3); g += kThreads) {
        const uint4 v = *reinterpret_cast<const uint4 *>(xr + g * 8);
        const uint32_t mb = (mask[g >> 2] >> ((g & 3) * 8)) & 0xFFu;
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
        uint32_t o[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const uint16_t lo = static_cast<uint16_t>(w[k] & 0xFFFFu), hi = static_cast<uint16_t>(w[k] >> 16);
          const uint16_t qlo = ((mb >> (2 * k)) & 1u) ? lo : fake(lo);
          const uint16_t qhi = ((mb >> (2 * k + 1)) & 1u) ? hi : fake(hi);
          o[k] = static_cast<uint32_t>(qlo) | (static_cast<uint32_t>(qhi) << 16);
        }
        *reinterpret_cast<uint4 *>(orow + g * 8) = make_uint4(o[0], o[1], o[2], o[3]);
      }
    } else {
      for (int64_t c = tid; c < cols; c += kThreads)
        orow[c] = ((mask[c >> 5] >> (c & 31)) & 1u) ? xr[c] : fake(xr[c]);
    }
  }
}

}  // namespace
}  // namespace quik

using namespace quik;

extern "C" int quik_sim_act_fake_quant(const void *x, int dtype, int64_t rows, int64_t cols, const uint32_t *outlier_mask,
                                       int bits, void *out, void *stream) {
  if (bits < 2 || bits > 8) return QUIK_ERR_BITS;
  if (dtype != QUIK_F16 && dtype != QUIK_BF16) return QUIK_ERR_DTYPE;
  if (rows < 0 || cols <= 0) return QUIK_ERR_SHAPE;
  if (rows == 0) return QUIK_OK;
  if (!x || !outlier_mask || !out) return QUIK_ERR_NULL;
  if (rows > (int64_t(1) << 31) || cols > (int64_t(1) << 31)) return QUIK_ERR_RANGE;
  const int vec = cols % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
  const int grid = static_cast<int>(rows < 65535 * 8 ? rows : 65535 * 8);
  const float maxq = static_cast<float>((1 << bits) - 1);
  if (dtype == QUIK_F16) {
    hipLaunchKernelGGL(act_fake_quant_kernel<false>, dim3(grid), dim3(kThreads), 0, as_stream(stream),
                       static_cast<const uint16_t *>(x), rows, cols, outlier_mask, maxq, static_cast<uint16_t *>(out), vec);
  } else {
    hipLaunchKernelGGL(act_fake_quant_kernel<true>, dim3(grid), dim3(kThreads), 0, as_stream(stream),
                       static_cast<const uint16_t *>(x), rows, cols, outlier_mask, maxq, static_cast<uint16_t *>(out), vec);
  }
  return check_launch();
}
