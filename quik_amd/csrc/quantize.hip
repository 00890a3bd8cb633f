// Per-token activation quantisation for MI355X (gfx950): column map, asymmetric quantize
// with outlier gather, find_meta, quantizeOld and the symmetric quantize.
//
// Arithmetic contract (what the parity tests pin bit for bit):
//   scale = storage(fmaxf((f32(max) - f32(min)) / (2^bits - 1), 1e-6f)), zero = min
//   d     = storage(x - zero)                     one rounding to fp16 / bf16
//   t     = storage(d / scale)                    correctly rounded quotient
//   v     = rne_int(t), NaN -> 0;  code = clamp(v, 0, 2^bits - 1) - 2^(bits-1)
// (reference: src/asymmetric/asymmetric.cu:340-435).
//
// Data flow of the asymmetric kernel, one 256-thread workgroup per row:
//   1. the row is streamed once from HBM with 16-byte loads into LDS; min/max are taken on
//      the fly over the non-outlier columns using one mask bit per column;
//   2. each lane then gathers two consecutive destination codes per step from LDS through a
//      compact source-column table, quantises them and stores one packed byte (int4) or two
//      bytes (int8); consecutive lanes hit consecutive LDS dwords and consecutive output bytes;
//   3. the outlier columns are gathered from LDS in the order the caller listed them.
// The quotient uses r = 1/scale (one IEEE division per row) and one Markstein correction
// step, q = d*r; e = fma(-q, s, d); q' = fma(e, r, q).  q' is within 2^-24(1+eps) of d/s
// relative, while d/s with 11-bit (8-bit for bf16) significands stays more than 2^-23
// relative away from every rounding boundary of the storage type, so storage(q') equals the
// correctly rounded storage(d/s).  Rows whose range overflows the storage type, or whose
// scale is below 1e-20 (bf16 only), take the plain IEEE division instead.
#include "common.h"

namespace quik {
namespace {

constexpr int kThreads = 256;

// ---------------------------------------------------------------------------------------
// column map layout: [src_col: num_int idx][fp_col: num_fp idx][mask: ceil(cols/32) u32]
// idx is uint16_t when cols <= 65536, else uint32_t.  Section offsets are 16-byte aligned.
struct ColmapLayout {
  bool idx16;
  int64_t off_fp, off_mask, bytes;
};

__host__ __device__ inline int64_t align16(int64_t v) { return (v + 15) & ~int64_t(15); }

__host__ __device__ inline ColmapLayout colmap_layout(int64_t cols, int64_t num_int, int64_t num_fp) {
  ColmapLayout l;
  l.idx16 = cols <= 65536;
  const int64_t isz = l.idx16 ? 2 : 4;
  l.off_fp = align16(num_int * isz);
  l.off_mask = l.off_fp + align16(num_fp * isz);
  l.bytes = l.off_mask + align16(((cols + 31) / 32) * 4);
  return l;
}

template <typename IdxT>
__global__ __launch_bounds__(1024) void colmap_build_kernel(const int64_t *__restrict__ int_idx, int64_t num_int,
                                                            const int64_t *__restrict__ fp_idx, int64_t num_fp,
                                                            int64_t cols, IdxT *__restrict__ src_col,
                                                            IdxT *__restrict__ fp_col, uint32_t *__restrict__ mask) {
  // single workgroup: the mask is cleared before any bit is set
  const int64_t words = (cols + 31) / 32;
  for (int64_t i = threadIdx.x; i < words; i += blockDim.x) mask[i] = 0u;
  __syncthreads();
  for (int64_t j = threadIdx.x; j < num_int; j += blockDim.x) {
    int64_t c = int_idx[j];
    c = c < 0 ? 0 : (c >= cols ? cols - 1 : c);
    src_col[j] = static_cast<IdxT>(c);
  }
  for (int64_t j = threadIdx.x; j < num_fp; j += blockDim.x) {
    int64_t c = fp_idx[j];
    c = c < 0 ? 0 : (c >= cols ? cols - 1 : c);
    fp_col[j] = static_cast<IdxT>(c);
    atomicOr(&mask[c >> 5], 1u << (c & 31));
  }
}

// ---------------------------------------------------------------------------------------
// block-wide (min, max) reduction; every thread returns the result
__device__ __forceinline__ void block_minmax(float &mn, float &mx, float *red) {
  mn = wave_min(mn);
  mx = wave_max(mx);
  const int wave = threadIdx.x >> 6;
  __syncthreads();  // protects `red` from the previous use
  if ((threadIdx.x & 63) == 0) {
    red[wave] = mn;
    red[4 + wave] = mx;
  }
  __syncthreads();
  mn = fminf(fminf(red[0], red[1]), fminf(red[2], red[3]));
  mx = fmaxf(fmaxf(red[4], red[5]), fmaxf(red[6], red[7]));
}

template <bool BF16>
struct RowQuant {
  float zero, scale, rcp;
  bool slow;
  uint16_t scale_bits, zero_bits;

  __device__ __forceinline__ void init(float mn, float mx, int bits) {
    if (!(mx >= mn)) {  // no non-NaN element in the row
      mn = mx = __builtin_nanf("");
    }
    const float range = mx - mn;
    const float s32 = fmaxf(range / static_cast<float>((1 << bits) - 1), 1e-6f);
    scale_bits = from_f32<BF16>(s32);
    zero_bits = from_f32<BF16>(mn);
    scale = to_f32<BF16>(scale_bits);
    zero = mn;
    rcp = 1.0f / scale;
    const float max_finite = BF16 ? 3.3895313892515355e38f : 65504.0f;
    slow = !(range <= max_finite) || !(scale >= 1e-20f);
  }

  // storage(storage(x - zero) / scale) as fp32
  __device__ __forceinline__ float quotient(uint16_t xbits) const {
    float d;
    if constexpr (BF16) {
      d = round_storage<true>(to_f32<true>(xbits) - zero);
    } else {
      const _Float16 dh = __builtin_bit_cast(_Float16, xbits) - static_cast<_Float16>(zero);
      d = static_cast<float>(dh);
    }
    float q;
    if (slow) {
      q = d / scale;
    } else {
      q = d * rcp;
      const float e = __builtin_fmaf(-q, scale, d);
      q = __builtin_fmaf(e, rcp, q);
    }
    return round_storage<BF16>(q);
  }

  // clamp(rne_int(t), 0, maxq), NaN -> 0, for maxq <= 255
  static __device__ __forceinline__ uint32_t to_level(float t, float maxq) {
    const float c = fminf(fmaxf(t, 0.0f), maxq);
    return __float_as_uint(c + 12582912.0f) & 0xFFu;  // 1.5 * 2^23: integer lands in the low mantissa bits
  }
};

template <typename IdxT, int BITS, bool BF16>
__global__ __launch_bounds__(kThreads) void asym_quantize_kernel(
    const uint16_t *__restrict__ x, int64_t rows, int64_t cols, const IdxT *__restrict__ src_col,
    const IdxT *__restrict__ fp_col, const uint32_t *__restrict__ mask, int64_t num_int, int64_t num_fp,
    uint8_t *__restrict__ dst, uint16_t *__restrict__ meta, uint16_t *__restrict__ fp_x, int vec_ok) {
  extern __shared__ __align__(16) uint16_t row_s[];
  __shared__ float red[8];
  const int tid = threadIdx.x;
  constexpr float kMaxQ = static_cast<float>((1 << BITS) - 1);
  constexpr uint32_t kFlip = BITS == 4 ? 0x88u : 0x8080u;

  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const uint16_t *xr = x + row * cols;
    float mn = __builtin_inff(), mx = -__builtin_inff();
    if (vec_ok) {
      const uint4 *xv = reinterpret_cast<const uint4 *>(xr);
      uint4 *sv = reinterpret_cast<uint4 *>(row_s);
      const int64_t nvec = cols >> 3;
      for (int64_t c8 = tid; c8 < nvec; c8 += kThreads) {
        const uint4 v = xv[c8];
        sv[c8] = v;
        uint32_t mb = (mask[c8 >> 2] >> ((c8 & 3) * 8)) & 0xFFu;
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float lo = to_f32<BF16>(static_cast<uint16_t>(w[i] & 0xFFFFu));
          const float hi = to_f32<BF16>(static_cast<uint16_t>(w[i] >> 16));
          if (!(mb & (1u << (2 * i)))) {
            mn = fminf(mn, lo);
            mx = fmaxf(mx, lo);
          }
          if (!(mb & (2u << (2 * i)))) {
            mn = fminf(mn, hi);
            mx = fmaxf(mx, hi);
          }
        }
      }
    } else {
      for (int64_t c = tid; c < cols; c += kThreads) {
        const uint16_t v = xr[c];
        row_s[c] = v;
        if (!((mask[c >> 5] >> (c & 31)) & 1u)) {
          const float f = to_f32<BF16>(v);
          mn = fminf(mn, f);
          mx = fmaxf(mx, f);
        }
      }
    }
    block_minmax(mn, mx, red);  // also orders the LDS row writes before the gathers below

    RowQuant<BF16> rq;
    rq.init(mn, mx, BITS);
    if (tid == 0) {
      meta[2 * row] = rq.scale_bits;
      meta[2 * row + 1] = rq.zero_bits;
    }

    const int64_t pairs = num_int >> 1;
    if constexpr (BITS == 4) {
      uint8_t *drow = dst + row * pairs;
      for (int64_t p = tid; p < pairs; p += kThreads) {
        const IdxT c0 = src_col[2 * p], c1 = src_col[2 * p + 1];
        const uint32_t v0 = RowQuant<BF16>::to_level(rq.quotient(row_s[c0]), kMaxQ);
        const uint32_t v1 = RowQuant<BF16>::to_level(rq.quotient(row_s[c1]), kMaxQ);
        drow[p] = static_cast<uint8_t>((v0 | (v1 << 4)) ^ kFlip);
      }
    } else {
      uint16_t *drow = reinterpret_cast<uint16_t *>(dst + row * num_int);
      for (int64_t p = tid; p < pairs; p += kThreads) {
        const IdxT c0 = src_col[2 * p], c1 = src_col[2 * p + 1];
        const uint32_t v0 = RowQuant<BF16>::to_level(rq.quotient(row_s[c0]), kMaxQ);
        const uint32_t v1 = RowQuant<BF16>::to_level(rq.quotient(row_s[c1]), kMaxQ);
        drow[p] = static_cast<uint16_t>((v0 | (v1 << 8)) ^ kFlip);
      }
    }
    uint16_t *frow = fp_x + row * num_fp;
    for (int64_t f = tid; f < num_fp; f += kThreads) frow[f] = row_s[fp_col[f]];
    __syncthreads();  // the next row overwrites row_s
  }
}

// Rows too long for LDS: same arithmetic, gathers go to global memory (L2-resident row).
template <typename IdxT, int BITS, bool BF16>
__global__ __launch_bounds__(kThreads) void asym_quantize_longrow_kernel(
    const uint16_t *__restrict__ x, int64_t rows, int64_t cols, const IdxT *__restrict__ src_col,
    const IdxT *__restrict__ fp_col, int64_t num_int, int64_t num_fp, uint8_t *__restrict__ dst,
    uint16_t *__restrict__ meta, uint16_t *__restrict__ fp_x) {
  __shared__ float red[8];
  const int tid = threadIdx.x;
  constexpr float kMaxQ = static_cast<float>((1 << BITS) - 1);
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const uint16_t *xr = x + row * cols;
    float mn = __builtin_inff(), mx = -__builtin_inff();
    for (int64_t j = tid; j < num_int; j += kThreads) {
      const float f = to_f32<BF16>(xr[src_col[j]]);
      mn = fminf(mn, f);
      mx = fmaxf(mx, f);
    }
    block_minmax(mn, mx, red);
    RowQuant<BF16> rq;
    rq.init(mn, mx, BITS);
    if (tid == 0) {
      meta[2 * row] = rq.scale_bits;
      meta[2 * row + 1] = rq.zero_bits;
    }
    const int64_t pairs = num_int >> 1;
    for (int64_t p = tid; p < pairs; p += kThreads) {
      const uint32_t v0 = RowQuant<BF16>::to_level(rq.quotient(xr[src_col[2 * p]]), kMaxQ);
      const uint32_t v1 = RowQuant<BF16>::to_level(rq.quotient(xr[src_col[2 * p + 1]]), kMaxQ);
      if constexpr (BITS == 4) {
        dst[row * pairs + p] = static_cast<uint8_t>((v0 | (v1 << 4)) ^ 0x88u);
      } else {
        reinterpret_cast<uint16_t *>(dst + row * num_int)[p] = static_cast<uint16_t>((v0 | (v1 << 8)) ^ 0x8080u);
      }
    }
    for (int64_t f = tid; f < num_fp; f += kThreads) fp_x[row * num_fp + f] = xr[fp_col[f]];
  }
}

// ---------------------------------------------------------------------------------------
// find_meta: fp16, all columns (reference: src/asymmetric/asymmetric.cu:263-338)
__global__ __launch_bounds__(kThreads) void find_meta_kernel(const uint16_t *__restrict__ x, int64_t rows,
                                                             int64_t cols, int bits, uint16_t *__restrict__ meta) {
  __shared__ float red[8];
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const uint16_t *xr = x + row * cols;
    float mn = __builtin_inff(), mx = -__builtin_inff();
    for (int64_t c = threadIdx.x; c < cols; c += kThreads) {
      const float f = to_f32<false>(xr[c]);
      mn = fminf(mn, f);
      mx = fmaxf(mx, f);
    }
    block_minmax(mn, mx, red);
    if (threadIdx.x == 0) {
      RowQuant<false> rq;
      rq.init(mn, mx, bits);
      meta[2 * row] = rq.scale_bits;
      meta[2 * row + 1] = rq.zero_bits;
    }
  }
}

__device__ __forceinline__ uint32_t old_level(uint16_t xb, uint16_t sb, uint16_t zb, float maxq) {
  const _Float16 d = __builtin_bit_cast(_Float16, xb) - __builtin_bit_cast(_Float16, zb);
  const float q = static_cast<float>(d) / static_cast<float>(__builtin_bit_cast(_Float16, sb));
  return RowQuant<false>::to_level(round_storage<false>(q), maxq);
}

// quantizeOld, 4 bit: flat pairing over the whole array, meta row = idx / colsDst
// (reference: src/asymmetric/asymmetric.cu:13-45)
__global__ __launch_bounds__(kThreads) void quantize_old4_kernel(const uint16_t *__restrict__ x,
                                                                 const uint16_t *__restrict__ meta, int64_t rows,
                                                                 int64_t cols, int64_t cols_dst,
                                                                 uint8_t *__restrict__ dst) {
  const int64_t n_dst = rows * cols_dst, n_src = rows * cols;
  for (int64_t idx = blockIdx.x * int64_t(kThreads) + threadIdx.x; idx < n_dst; idx += int64_t(gridDim.x) * kThreads) {
    const int64_t row = idx / cols_dst;
    const uint16_t sb = meta[2 * row], zb = meta[2 * row + 1];
    uint32_t byte = 0;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int64_t s = idx * 2 + i;
      if (s < n_src) byte |= ((old_level(x[s], sb, zb, 15.0f) ^ 8u) & 0xFu) << (4 * i);
    }
    dst[idx] = static_cast<uint8_t>(byte);
  }
}

__global__ __launch_bounds__(kThreads) void quantize_old8_kernel(const uint16_t *__restrict__ x,
                                                                 const uint16_t *__restrict__ meta, int64_t rows,
                                                                 int64_t cols, uint8_t *__restrict__ dst) {
  const int64_t n = rows * cols;
  for (int64_t idx = blockIdx.x * int64_t(kThreads) + threadIdx.x; idx < n; idx += int64_t(gridDim.x) * kThreads) {
    const int64_t row = idx / cols;
    dst[idx] = static_cast<uint8_t>(old_level(x[idx], meta[2 * row], meta[2 * row + 1], 255.0f) ^ 0x80u);
  }
}

// symmetric quantize (reference: src/symmetric/symmetric.cu:6-61): no clamp, wraps
__device__ __forceinline__ int sym_code(uint16_t xb, float s) {
  const float q = round_storage<false>(to_f32<false>(xb) / s);
  // __half2int_rn: NaN -> 0, saturating
  return __float2int_rn(q);
}

__global__ __launch_bounds__(kThreads) void sym_quantize_kernel(const uint16_t *__restrict__ x,
                                                                const uint16_t *__restrict__ scale, int64_t rows,
                                                                int64_t cols, int bits, uint8_t *__restrict__ dst) {
  const int64_t cols_dst = bits == 4 ? (cols + 1) / 2 : cols;
  for (int64_t row = blockIdx.y; row < rows; row += gridDim.y) {
    const float s = to_f32<false>(scale[row]);
    const uint16_t *xr = x + row * cols;
    uint8_t *dr = dst + row * cols_dst;
    for (int64_t j = blockIdx.x * int64_t(kThreads) + threadIdx.x; j < cols_dst; j += int64_t(gridDim.x) * kThreads) {
      if (bits == 4) {
        uint32_t b = static_cast<uint32_t>(sym_code(xr[2 * j], s)) & 0xFu;
        if (2 * j + 1 < cols) b |= (static_cast<uint32_t>(sym_code(xr[2 * j + 1], s)) & 0xFu) << 4;
        dr[j] = static_cast<uint8_t>(b);
      } else {
        dr[j] = static_cast<uint8_t>(sym_code(xr[j], s) & 0xFF);
      }
    }
  }
}

int grid_for(int64_t work_items, int64_t per_block) {
  int64_t g = (work_items + per_block - 1) / per_block;
  if (g < 1) g = 1;
  if (g > 65535 * 16) g = 65535 * 16;
  return static_cast<int>(g);
}

constexpr int64_t kMaxLdsRowBytes = 128 * 1024;  // of the 160 KB per CU

template <typename IdxT, int BITS, bool BF16>
int launch_asym(const void *x, int64_t rows, int64_t cols, const uint8_t *cm, const ColmapLayout &l, int64_t num_int,
                int64_t num_fp, void *dst, void *meta, void *fp_x, hipStream_t st) {
  const IdxT *src_col = reinterpret_cast<const IdxT *>(cm);
  const IdxT *fp_col = reinterpret_cast<const IdxT *>(cm + l.off_fp);
  const uint32_t *mask = reinterpret_cast<const uint32_t *>(cm + l.off_mask);
  const int grid = static_cast<int>(rows < 65535 * 8 ? rows : 65535 * 8);
  const int64_t lds = align16(cols * 2);
  if (lds <= kMaxLdsRowBytes) {
    auto kern = asym_quantize_kernel<IdxT, BITS, BF16>;
    if (lds > 48 * 1024) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
      if (e != hipSuccess) {
        set_last_hip_error(e);
        return QUIK_ERR_LAUNCH;
      }
    }
    const int vec_ok = (cols % 8 == 0) && (reinterpret_cast<uintptr_t>(x) % 16 == 0);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), static_cast<size_t>(lds), st,
                       static_cast<const uint16_t *>(x), rows, cols, src_col, fp_col, mask, num_int, num_fp,
                       static_cast<uint8_t *>(dst), static_cast<uint16_t *>(meta), static_cast<uint16_t *>(fp_x),
                       vec_ok);
  } else {
    hipLaunchKernelGGL((asym_quantize_longrow_kernel<IdxT, BITS, BF16>), dim3(grid), dim3(kThreads), 0, st,
                       static_cast<const uint16_t *>(x), rows, cols, src_col, fp_col, num_int, num_fp,
                       static_cast<uint8_t *>(dst), static_cast<uint16_t *>(meta), static_cast<uint16_t *>(fp_x));
  }
  return check_launch();
}

}  // namespace
}  // namespace quik

using namespace quik;

extern "C" int64_t quik_colmap_bytes(int64_t cols, int64_t num_int, int64_t num_fp) {
  if (cols <= 0 || num_int < 0 || num_fp < 0 || num_int + num_fp != cols) return 0;
  return colmap_layout(cols, num_int, num_fp).bytes;
}

extern "C" int quik_colmap_build(const int64_t *int_indices, int64_t num_int, const int64_t *fp_indices,
                                 int64_t num_fp, int64_t cols, void *colmap, void *stream) {
  if (cols <= 0 || num_int < 0 || num_fp < 0 || num_int + num_fp != cols) return QUIK_ERR_SHAPE;
  if (!colmap || (num_int > 0 && !int_indices) || (num_fp > 0 && !fp_indices)) return QUIK_ERR_NULL;
  if (cols > (int64_t(1) << 31)) return QUIK_ERR_RANGE;
  const ColmapLayout l = colmap_layout(cols, num_int, num_fp);
  uint8_t *cm = static_cast<uint8_t *>(colmap);
  uint32_t *mask = reinterpret_cast<uint32_t *>(cm + l.off_mask);
  if (l.idx16) {
    hipLaunchKernelGGL(colmap_build_kernel<uint16_t>, dim3(1), dim3(1024), 0, as_stream(stream), int_indices,
                       num_int, fp_indices, num_fp, cols, reinterpret_cast<uint16_t *>(cm),
                       reinterpret_cast<uint16_t *>(cm + l.off_fp), mask);
  } else {
    hipLaunchKernelGGL(colmap_build_kernel<uint32_t>, dim3(1), dim3(1024), 0, as_stream(stream), int_indices,
                       num_int, fp_indices, num_fp, cols, reinterpret_cast<uint32_t *>(cm),
                       reinterpret_cast<uint32_t *>(cm + l.off_fp), mask);
  }
  return check_launch();
}

extern "C" int quik_asym_quantize(const void *x, int dtype, int64_t rows, int64_t cols, const void *colmap,
                                  int64_t num_int, int64_t num_fp, int bits, void *dst, void *meta, void *fp_x,
                                  void *stream) {
  if (bits != 4 && bits != 8) return QUIK_ERR_BITS;
  if (dtype != QUIK_F16 && dtype != QUIK_BF16) return QUIK_ERR_DTYPE;
  if (rows < 0 || cols <= 0 || num_int <= 0 || num_fp < 0 || num_int + num_fp != cols) return QUIK_ERR_SHAPE;
  if (num_int % 2 != 0) return QUIK_ERR_ALIGN;
  if (rows == 0) return QUIK_OK;
  if (!x || !colmap || !dst || !meta || (num_fp > 0 && !fp_x)) return QUIK_ERR_NULL;
  if (cols > (int64_t(1) << 31)) return QUIK_ERR_RANGE;
  const ColmapLayout l = colmap_layout(cols, num_int, num_fp);
  const uint8_t *cm = static_cast<const uint8_t *>(colmap);
  hipStream_t st = as_stream(stream);
#define QUIK_DISPATCH(IDX)                                                                                     \
  if (bits == 4) {                                                                                             \
    return dtype == QUIK_F16                                                                                   \
               ? launch_asym<IDX, 4, false>(x, rows, cols, cm, l, num_int, num_fp, dst, meta, fp_x, st)       \
               : launch_asym<IDX, 4, true>(x, rows, cols, cm, l, num_int, num_fp, dst, meta, fp_x, st);       \
  } else {                                                                                                     \
    return dtype == QUIK_F16                                                                                   \
               ? launch_asym<IDX, 8, false>(x, rows, cols, cm, l, num_int, num_fp, dst, meta, fp_x, st)       \
               : launch_asym<IDX, 8, true>(x, rows, cols, cm, l, num_int, num_fp, dst, meta, fp_x, st);       \
  }
  if (l.idx16) {
    QUIK_DISPATCH(uint16_t)
  } else {
    QUIK_DISPATCH(uint32_t)
  }
#undef QUIK_DISPATCH
}

extern "C" int quik_asym_find_meta(const void *x, int64_t rows, int64_t cols, int bits, void *meta, void *stream) {
  if (bits != 4 && bits != 8) return QUIK_ERR_BITS;
  if (rows < 0 || cols <= 0) return QUIK_ERR_SHAPE;
  if (rows == 0) return QUIK_OK;
  if (!x || !meta) return QUIK_ERR_NULL;
  const int grid = static_cast<int>(rows < 65535 ? rows : 65535);
  hipLaunchKernelGGL(find_meta_kernel, dim3(grid), dim3(kThreads), 0, as_stream(stream),
                     static_cast<const uint16_t *>(x), rows, cols, bits, static_cast<uint16_t *>(meta));
  return check_launch();
}

extern "C" int quik_asym_quantize_old(const void *x, const void *meta, int64_t rows, int64_t cols, int bits,
                                      void *dst, void *stream) {
  if (bits != 4 && bits != 8) return QUIK_ERR_BITS;
  if (rows < 0 || cols <= 0) return QUIK_ERR_SHAPE;
  if (rows == 0) return QUIK_OK;
  if (!x || !meta || !dst) return QUIK_ERR_NULL;
  if (bits == 4) {
    const int64_t cols_dst = (cols + 1) / 2;
    hipLaunchKernelGGL(quantize_old4_kernel, dim3(grid_for(rows * cols_dst, kThreads * 4)), dim3(kThreads), 0,
                       as_stream(stream), static_cast<const uint16_t *>(x), static_cast<const uint16_t *>(meta), rows,
                       cols, cols_dst, static_cast<uint8_t *>(dst));
  } else {
    hipLaunchKernelGGL(quantize_old8_kernel, dim3(grid_for(rows * cols, kThreads * 4)), dim3(kThreads), 0,
                       as_stream(stream), static_cast<const uint16_t *>(x), static_cast<const uint16_t *>(meta), rows,
                       cols, static_cast<uint8_t *>(dst));
  }
  return check_launch();
}

extern "C" int quik_sym_quantize(const void *x, const void *scale, int64_t rows, int64_t cols, int bits, void *dst,
                                 void *stream) {
  if (bits != 4 && bits != 8) return QUIK_ERR_BITS;
  if (rows < 0 || cols <= 0) return QUIK_ERR_SHAPE;
  if (rows == 0) return QUIK_OK;
  if (!x || !scale || !dst) return QUIK_ERR_NULL;
  const int64_t cols_dst = bits == 4 ? (cols + 1) / 2 : cols;
  int gx = grid_for(cols_dst, kThreads);
  if (gx > 64) gx = 64;
  const int gy = static_cast<int>(rows < 65535 ? rows : 65535);
  hipLaunchKernelGGL(sym_quantize_kernel, dim3(gx, gy), dim3(kThreads), 0, as_stream(stream),
                     static_cast<const uint16_t *>(x), static_cast<const uint16_t *>(scale), rows, cols, bits,
                     static_cast<uint8_t *>(dst));
  return check_launch();
}
