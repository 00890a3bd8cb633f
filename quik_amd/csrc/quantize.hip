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
// Two kernels implement it.  The streaming kernel (see "Streaming path" below) serves the usual
// layout, ascending int_indices; the gather kernel serves any other order: it copies the row
// to LDS with 16-byte loads while taking min/max over the non-outlier columns (one mask bit per
// column), then each lane gathers two consecutive destination codes per step from LDS through a
// compact source-column table and stores one packed byte (int4) or two bytes (int8).
//
// The quotient.  r = 1/scale is one IEEE division per row.  The gather kernel and the bf16
// streaming path use q = d*r; e = fma(-q, s, d); q' = fma(e, r, q): q' is within
// 2^-24(1+eps) of d/s relative, while d/s with 11-bit (8-bit for bf16) significands stays more
// than 2^-23 relative away from every rounding boundary of the storage type, so storage(q')
// equals the correctly rounded storage(d/s).  The fp16 streaming path uses fp16(d*r) without
// the correction step: that value can differ from storage(d/s) in the last place (about 1.5e-6
// of all (d, s) pairs) but never across a k + 1/2 boundary, so rne_int gives the same level for
// every fp16 d >= 0 and every fp16 scale >= 1e-6 with both 4 and 8 bits; the tests enumerate
// that whole domain.  Rows whose range overflows the storage type, or whose scale is below
// 1e-20 (bf16 only), take the plain IEEE division instead.
#include <type_traits>

#include "colmap.h"
#include "common.h"
#include "fp6_format.h"
#include "quantize_math.h"

namespace quik {
namespace {

constexpr int kThreads = 256;

// number of non-zero bytes among the low `nbytes` bytes of w
__device__ __forceinline__ uint32_t nonzero_bytes(uint32_t w, int nbytes) {
  uint32_t n = 0;
  for (int b = 0; b < nbytes; ++b) n += ((w >> (8 * b)) & 0xFFu) != 0u;
  return n;
}

template <typename IdxT>
__global__ __launch_bounds__(1024) void colmap_build_kernel(const int64_t *__restrict__ int_idx, int64_t num_int,
                                                            const int64_t *__restrict__ fp_idx, int64_t num_fp,
                                                            int64_t cols, IdxT *__restrict__ src_col,
                                                            IdxT *__restrict__ fp_col, uint32_t *__restrict__ mask,
                                                            uint32_t *__restrict__ grp, uint32_t *__restrict__ dirty,
                                                            uint16_t *__restrict__ dirty_grp,
                                                            uint16_t *__restrict__ kperm, uint32_t *__restrict__ patch,
                                                            uint16_t *__restrict__ unit, uint16_t *__restrict__ gather_unit,
                                                            uint16_t *__restrict__ gather_cols,
                                                            uint32_t *__restrict__ flags) {
  // single workgroup: the mask is cleared before any bit is set
  __shared__ int ascending;
  __shared__ uint32_t prefix[kStreamMaxCols / 32 + 1];  // outliers in columns [0, 32 w)
  if (threadIdx.x == 0) ascending = 1;
  const int64_t words = (cols + 31) / 32;
  for (int64_t i = threadIdx.x; i < words; i += blockDim.x) mask[i] = 0u;
  __syncthreads();
  for (int64_t j = threadIdx.x; j < num_int; j += blockDim.x) {
    int64_t c = int_idx[j];
    if (j + 1 < num_int && !(c < int_idx[j + 1])) ascending = 0;
    if (c < 0 || c >= cols) ascending = 0;
    c = c < 0 ? 0 : (c >= cols ? cols - 1 : c);
    src_col[j] = static_cast<IdxT>(c);
  }
  for (int64_t j = threadIdx.x; j < num_fp; j += blockDim.x) {
    int64_t c = fp_idx[j];
    c = c < 0 ? 0 : (c >= cols ? cols - 1 : c);
    fp_col[j] = static_cast<IdxT>(c);
    atomicOr(&mask[c >> 5], 1u << (c & 31));
  }
  __syncthreads();
  // the two lists must not share a column (the streaming kernels take the integer columns as the complement of
  // the outlier mask, the gather kernels take them from src_col: they agree only for a partition)
  for (int64_t j = threadIdx.x; j < num_int; j += blockDim.x) {
    const int64_t c = int_idx[j];
    if (c >= 0 && c < cols && ((mask[c >> 5] >> (c & 31)) & 1u)) ascending = 0;
  }
  __syncthreads();
  const bool stream_shape = cols <= kStreamMaxCols && cols % 8 == 0;
  // ascending int_indices (strictly, in range, none of them an outlier column) and num_fp distinct outlier
  // columns, num_int + num_fp == cols: a partition
  uint32_t total = 0, total_dirty = 0;
  if (threadIdx.x == 0) {
    for (int64_t w = 0; w < words; ++w) {
      total += __popc(mask[w]);
      total_dirty += nonzero_bytes(mask[w], 4);
    }
    const bool streams = ascending && stream_shape && total == num_fp;
    const bool in_place = streams && num_int % 32 == 0 && num_fp % 32 == 0;
    flags[0] = (streams ? 1u : 0u) | (in_place ? 2u : 0u);
    flags[1] = total_dirty;
    flags[2] = flags[3] = 0u;
    if (cols <= kStreamMaxCols) {
      uint32_t run = 0;
      for (int64_t w = 0; w < words; ++w) {
        prefix[w] = run;
        run += __popc(mask[w]);
      }
      prefix[words] = run;
    }
  }
  __syncthreads();
  if (cols <= kStreamMaxCols && (flags[0] & 2u)) {
    // outliers in columns [0, c)
    auto before = [&](int64_t c) {
      return prefix[c >> 5] + ((c & 31) ? __popc(mask[c >> 5] & ((1u << (c & 31)) - 1u)) : 0);
    };
    auto is_outlier = [&](int64_t c) { return (mask[c >> 5] >> (c & 31)) & 1u; };
    const uint32_t holes = before(num_int);   // = integer columns in the tail
    if (threadIdx.x == 0) flags[2] = holes;
    uint16_t *hole_col = reinterpret_cast<uint16_t *>(patch), *filler_col = hole_col + 1;  // interleaved halves
    for (int64_t c = threadIdx.x; c < cols; c += blockDim.x) {
      const uint32_t ob = before(c);
      if (c < num_int) {
        if (is_outlier(c)) {
          hole_col[2 * ob] = static_cast<uint16_t>(c);
        } else {
          kperm[c] = static_cast<uint16_t>(c - ob);
        }
      } else if (!is_outlier(c)) {
        filler_col[2 * ((c - num_int) - (ob - holes))] = static_cast<uint16_t>(c);
      }
    }
    __syncthreads();
    for (int64_t i = threadIdx.x; i < holes; i += blockDim.x) {
      const int64_t f = filler_col[2 * i];
      kperm[hole_col[2 * i]] = static_cast<uint16_t>(f - before(f));
    }
  }
  if (cols <= kStreamMaxCols) {
    const int64_t groups = (cols + 7) / 8;
    const int64_t cap = max_dirty_groups(cols, num_fp);
    for (int64_t g = threadIdx.x; g < groups; g += blockDim.x) {
      uint32_t before = 0, slot = 0;
      for (int64_t w = 0; w < (g >> 2); ++w) {
        before += __popc(mask[w]);
        slot += nonzero_bytes(mask[w], 4);
      }
      const uint32_t word = mask[g >> 2];
      const int sh = static_cast<int>(g & 3) * 8;
      before += __popc(word & ((1u << sh) - 1u));
      slot += nonzero_bytes(word, static_cast<int>(g & 3));
      const uint32_t mb = (word >> sh) & 0xFFu;
      const uint32_t dest = static_cast<uint32_t>(g * 8) - before;
      if (mb == 0u) {
        grp[g] = dest << 8;
      } else {
        grp[g] = (slot << 8) | mb;
        if (slot < cap) {
          dirty[slot] = (dest << 8) | mb;
          dirty_grp[slot] = static_cast<uint16_t>(g);
        }
      }
    }
  }
  // 16-column units of the tile-ordered int8 operand buffers (colmap.h)
  if (cols <= kStreamMaxCols && (flags[0] & 1u) && num_int % 16 == 0) {
    const int64_t units = num_int / 16;
    for (int64_t u = threadIdx.x; u < units; u += blockDim.x) {
      const uint32_t c0 = src_col[16 * u], c15 = src_col[16 * u + 15];
      unit[u] = c15 - c0 == 15u ? static_cast<uint16_t>(c0) : uint16_t(0xFFFF);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      uint32_t n = 0;
      for (int64_t u = 0; u < units; ++u) {
        if (unit[u] != 0xFFFFu) continue;
        if (n < num_fp) {  // (always: an outlier column lies inside the span of at most one unit)
          gather_unit[n] = static_cast<uint16_t>(u);
          for (int t = 0; t < 16; ++t) gather_cols[16 * n + t] = static_cast<uint16_t>(src_col[16 * u + t]);
        }
        ++n;
      }
      flags[3] = n;
    }
  }
}

// ---------------------------------------------------------------------------------------
// block-wide (min, max) reduction; every thread returns the result
template <int TPR = kThreads>
__device__ __forceinline__ void block_minmax(float &mn, float &mx, float *red) {
  mn = wave_min(mn);
  mx = wave_max(mx);
  __syncthreads();  // protects `red` from the previous use (and orders the callers' LDS row writes)
  if constexpr (TPR > 64) {
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) {
      red[wave] = mn;
      red[4 + wave] = mx;
    }
    __syncthreads();
    mn = red[0];
    mx = red[4];
#pragma unroll
    for (int w = 1; w < TPR / 64; ++w) {
      mn = fminf(mn, red[w]);
      mx = fmaxf(mx, red[4 + w]);
    }
  }
}

template <typename IdxT, int BITS, bool BF16, int TPR = kThreads>
__device__ __forceinline__ void gather_rows(
    const uint16_t *__restrict__ x, int64_t rows, int64_t cols, const IdxT *__restrict__ src_col,
    const IdxT *__restrict__ fp_col, const uint32_t *__restrict__ mask, int64_t num_int, int64_t num_fp,
    uint8_t *__restrict__ dst, uint16_t *__restrict__ meta, uint16_t *__restrict__ fp_x, int vec_ok,
    uint16_t *row_s, float *red) {
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
      for (int64_t c8 = tid; c8 < nvec; c8 += TPR) {
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
      for (int64_t c = tid; c < cols; c += TPR) {
        const uint16_t v = xr[c];
        row_s[c] = v;
        if (!((mask[c >> 5] >> (c & 31)) & 1u)) {
          const float f = to_f32<BF16>(v);
          mn = fminf(mn, f);
          mx = fmaxf(mx, f);
        }
      }
    }
    block_minmax<TPR>(mn, mx, red);  // also orders the LDS row writes before the gathers below

    RowQuant<BF16> rq;
    rq.init(mn, mx, BITS);
    if (tid == 0) {
      meta[2 * row] = rq.scale_bits;
      meta[2 * row + 1] = rq.zero_bits;
    }

    const int64_t pairs = num_int >> 1;
    if constexpr (BITS == 4) {
      uint8_t *drow = dst + row * pairs;
      for (int64_t p = tid; p < pairs; p += TPR) {
        const IdxT c0 = src_col[2 * p], c1 = src_col[2 * p + 1];
        const uint32_t v0 = RowQuant<BF16>::to_level(rq.quotient(row_s[c0]), kMaxQ);
        const uint32_t v1 = RowQuant<BF16>::to_level(rq.quotient(row_s[c1]), kMaxQ);
        drow[p] = static_cast<uint8_t>((v0 | (v1 << 4)) ^ kFlip);
      }
    } else {
      uint16_t *drow = reinterpret_cast<uint16_t *>(dst + row * num_int);
      for (int64_t p = tid; p < pairs; p += TPR) {
        const IdxT c0 = src_col[2 * p], c1 = src_col[2 * p + 1];
        const uint32_t v0 = RowQuant<BF16>::to_level(rq.quotient(row_s[c0]), kMaxQ);
        const uint32_t v1 = RowQuant<BF16>::to_level(rq.quotient(row_s[c1]), kMaxQ);
        drow[p] = static_cast<uint16_t>((v0 | (v1 << 8)) ^ kFlip);
      }
    }
    if (fp_x != nullptr) {
      uint16_t *frow = fp_x + row * num_fp;
      for (int64_t f = tid; f < num_fp; f += TPR) frow[f] = row_s[fp_col[f]];
    }
    __syncthreads();  // the next row overwrites row_s
  }
}

// ---------------------------------------------------------------------------------------
// Streaming path (ascending int_indices, the layout MixedQLinear.from_float produces).
//
// Works in source order, so nothing is gathered.  Every lane keeps NV 16-byte groups of the row
// in registers.
// All lanes run the same branch-free code on their groups as if they were clean: packed fp16
// min/max (a dirty group's contribution is replaced by the neutral element with one select),
// then 8 codes per group, written as 8 bytes to the group's destination position in an LDS byte
// buffer (only that write is predicated).  Dirty groups are handled a second time by lanes
// 0..ndirty-1, one group each, with per-element masking: that keeps the expensive masked code off
// the all-lanes path, where a divergent branch would make every wave pay for both sides.  Those
// lanes load their group (and every lane its outlier value) straight from the row, right after
// the row's own loads, so the data arrives with them (same cache lines).  A last pass reads 16
// code bytes per lane, packs them to nibbles (int4) and writes 8 or 16 contiguous bytes per lane.
// One row is handled by the TPR threads of one workgroup (a multiple of 64, at most 256; the
// launches use 256), which walks over rows blockIdx.x, blockIdx.x + gridDim.x, ...
// SYM: symmetric activations (scale = fp16(max |x| / sym_divisor), one scale per row in meta[row]); fp16 only.
template <int BITS, bool BF16, int NV, int TPR, bool SYM = false, bool PF = false>
__device__ __forceinline__ void stream_rows(const uint16_t *__restrict__ x, int64_t rows, int64_t cols,
                                            const uint32_t *__restrict__ grp, const uint32_t *__restrict__ dirty,
                                            const uint16_t *__restrict__ dirty_grp, int ndirty,
                                            const uint16_t *__restrict__ fp_col, int64_t num_int, int64_t num_fp,
                                            uint8_t *__restrict__ dst, uint16_t *__restrict__ meta,
                                            uint16_t *__restrict__ fp_x, uint8_t *codes_s, float *red, int vec_out,
                                            float sym_divisor = 1.0f) {
  // vec_out: 0 byte-wise output, 1 16-byte output,
  // 3 (8 bits only): dst is an int8 operand buffer in tile order for gemm_tile8.h, which also takes the outlier
  // values (fp_x is not written); needs num_int % 64 == 0 and num_fp % 32 == 0
  // (the 6-bit operand buffers of gemm_fp6.h are written by quantize_fp6_wave_kernel below)
  const Tile8Layout l8 = tile8_layout(rows, num_int, num_fp);
  const bool to8 = BITS == 8 && vec_out == 3;
  const int tid = threadIdx.x;
  const int nvec = static_cast<int>(cols >> 3);
  const float inf = __builtin_inff();
  // Row-invariant tables in registers.  Every load is unconditional, from an address that always exists (lanes
  // without an entry read the first words of grp): behind a condition each load sits in a branch of its own with
  // its own wait, and the kernel starts with one round trip to the L2 after the other.
  uint32_t g[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) g[i] = grp[tid + i * TPR < nvec ? tid + i * TPR : 0];
#pragma unroll
  for (int i = 0; i < NV; ++i) g[i] = tid + i * TPR < nvec ? g[i] : 0xFFFFFFFFu;
  // this lane's first ND dirty groups and outliers, so that the per-row loops below wait on no global load
  constexpr int ND = TPR >= 256 ? 1 : 256 / TPR;
  uint32_t my_dirty[ND], my_dgrp[ND], my_fpcol[ND];
  const uint16_t *spare16 = reinterpret_cast<const uint16_t *>(grp);
#pragma unroll
  for (int k = 0; k < ND; ++k) {
    const bool has_d = tid + k * TPR < ndirty, has_f = tid + k * TPR < num_fp;
    my_dirty[k] = *(has_d ? dirty + tid + k * TPR : grp);
    my_dgrp[k] = *(has_d ? dirty_grp + tid + k * TPR : spare16);
    my_fpcol[k] = *(has_f ? fp_col + tid + k * TPR : spare16);
  }
#pragma unroll
  for (int k = 0; k < ND; ++k) {
    if (!(tid + k * TPR < ndirty)) my_dirty[k] = my_dgrp[k] = 0u;
    if (!(tid + k * TPR < num_fp)) my_fpcol[k] = 0u;
  }

  auto load_row = [&](int64_t row, uint4 (&v)[NV]) {
    const uint4 *xv = reinterpret_cast<const uint4 *>(x + row * cols);
#pragma unroll
    for (int i = 0; i < NV; ++i) v[i] = xv[tid + i * TPR < nvec ? tid + i * TPR : nvec - 1];  // (past the end: any group; its g[i] says "not clean")
  };

  // min/max of one dirty group.  fp16: the outlier halves are overwritten with 0xFFFF, a quiet NaN,
  // which the packed min/max skip; bf16: per-element selects on fp32
  auto dirty_minmax = [&](const uint4 &v, uint32_t mb, h2 &pmn, h2 &pmx, float &mn, float &mx) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    if constexpr (!BF16) {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_sbfe(static_cast<int>(mb), 2 * k, 1));
        const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_sbfe(static_cast<int>(mb), 2 * k + 1, 1));
        const h2 m = __builtin_bit_cast(h2, w[k] | __builtin_amdgcn_perm(hi, lo, 0x07060100u));
        pmn = __builtin_elementwise_min(pmn, m);
        pmx = __builtin_elementwise_max(pmx, m);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float f = to_f32<true>(static_cast<uint16_t>(w[e >> 1] >> (16 * (e & 1))));
        const bool out = (mb >> e) & 1u;
        mn = fminf(mn, out ? inf : f);
        mx = fmaxf(mx, out ? -inf : f);
      }
    }
  };
  // SYM: largest |x| pattern of one dirty group, outlier halves zeroed
  auto dirty_absmax = [&](const uint4 &v, uint32_t mb, u2 &amax) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_sbfe(static_cast<int>(mb), 2 * k, 1));
      const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_sbfe(static_cast<int>(mb), 2 * k + 1, 1));
      const uint32_t outl = __builtin_amdgcn_perm(hi, lo, 0x07060100u);  // 0xFFFF in the outlier halves
      amax = __builtin_elementwise_max(amax, __builtin_bit_cast(u2, w[k] & 0x7FFF7FFFu & ~outl));
    }
  };
  // codes of one dirty group, outliers squeezed out
  auto dirty_codes = [&](const uint4 &v, uint32_t info, const RowQuant<BF16> &rq, auto slow_c) {
    constexpr bool SLOW = decltype(slow_c)::value;
    const uint32_t mb = info & 0xFFu;
    const uint2 c = group_codes<BITS, BF16, SLOW, SYM>(v, rq);
    uint8_t *out = codes_s + (info >> 8);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if (!((mb >> e) & 1u))
        out[e - __popc(mb & ((1u << e) - 1u))] = static_cast<uint8_t>((e < 4 ? c.x : c.y) >> (8 * (e & 3)));
    }
  };

  // one row; `cur` holds its groups, `parity` alternates so that two sets of reduction slots are used
  auto process = [&](int64_t row, const uint4 (&cur)[NV], const uint4 (&dv)[ND], const uint16_t (&fpv)[ND],
                     int parity) {
    const uint4 *xv = reinterpret_cast<const uint4 *>(x + row * cols);
    // ---- all lanes: min / max as if every group were clean
    float mn = inf, mx = -inf;
    const h2 pinf = h2{static_cast<_Float16>(inf), static_cast<_Float16>(inf)};
    h2 pmn = pinf, pmx = -pinf;
    u2 amax = u2{0, 0};  // SYM: largest |x| bit pattern per half (non-negative fp16 patterns order like unsigned integers)
    if constexpr (SYM) {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const u2 a = __builtin_bit_cast(u2, cur[i].x & 0x7FFF7FFFu), b = __builtin_bit_cast(u2, cur[i].y & 0x7FFF7FFFu);
        const u2 c = __builtin_bit_cast(u2, cur[i].z & 0x7FFF7FFFu), d = __builtin_bit_cast(u2, cur[i].w & 0x7FFF7FFFu);
        const u2 hi = __builtin_elementwise_max(__builtin_elementwise_max(a, b), __builtin_elementwise_max(c, d));
        const bool clean = (g[i] & 0xFFu) == 0u;
        amax = __builtin_elementwise_max(amax, clean ? hi : u2{0, 0});
      }
    } else if constexpr (!BF16) {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const h2 a = __builtin_bit_cast(h2, cur[i].x), b = __builtin_bit_cast(h2, cur[i].y);
        const h2 c = __builtin_bit_cast(h2, cur[i].z), d = __builtin_bit_cast(h2, cur[i].w);
        const h2 lo = __builtin_elementwise_min(__builtin_elementwise_min(a, b), __builtin_elementwise_min(c, d));
        const h2 hi = __builtin_elementwise_max(__builtin_elementwise_max(a, b), __builtin_elementwise_max(c, d));
        const bool clean = (g[i] & 0xFFu) == 0u;
        pmn = __builtin_elementwise_min(pmn, clean ? lo : pinf);
        pmx = __builtin_elementwise_max(pmx, clean ? hi : -pinf);
      }
    } else {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const uint32_t w[4] = {cur[i].x, cur[i].y, cur[i].z, cur[i].w};
        float lo = inf, hi = -inf;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const float f0 = __uint_as_float(w[k] << 16), f1 = __uint_as_float(w[k] & 0xFFFF0000u);
          lo = fminf(lo, fminf(f0, f1));
          hi = fmaxf(hi, fmaxf(f0, f1));
        }
        const bool clean = (g[i] & 0xFFu) == 0u;
        mn = fminf(mn, clean ? lo : inf);
        mx = fmaxf(mx, clean ? hi : -inf);
      }
    }
    // ---- outliers, in the caller's order
    auto fp_slot = [&](int64_t f) -> uint16_t * {
      if (to8)
        return reinterpret_cast<uint16_t *>(dst + tile8_offset(l8, row, l8.steps + (f >> 4), static_cast<int>((f >> 3) & 1))) + (f & 7);
      return fp_x + row * num_fp + f;
    };
#pragma unroll
    for (int k = 0; k < ND; ++k)
      if (tid + k * TPR < num_fp) *fp_slot(tid + k * TPR) = fpv[k];
    for (int64_t f = tid + ND * TPR; f < num_fp; f += TPR) *fp_slot(f) = x[row * cols + fp_col[f]];
    // ---- lanes 0 .. ndirty-1: one dirty group each (more when there are more than ND * TPR of them)
    if constexpr (SYM) {
#pragma unroll
      for (int k = 0; k < ND; ++k)
        if (tid + k * TPR < ndirty) dirty_absmax(dv[k], my_dirty[k] & 0xFFu, amax);
      for (int j = tid + ND * TPR; j < ndirty; j += TPR) dirty_absmax(xv[dirty_grp[j]], dirty[j] & 0xFFu, amax);
      mn = 0.0f;
      mx = static_cast<float>(amax.x > amax.y ? amax.x : amax.y);  // a 15-bit integer: exact, ordered like the patterns
    } else {
#pragma unroll
      for (int k = 0; k < ND; ++k)
        if (tid + k * TPR < ndirty) dirty_minmax(dv[k], my_dirty[k] & 0xFFu, pmn, pmx, mn, mx);
      for (int j = tid + ND * TPR; j < ndirty; j += TPR)
        dirty_minmax(xv[dirty_grp[j]], dirty[j] & 0xFFu, pmn, pmx, mn, mx);
      if constexpr (!BF16) {
        mn = fminf(static_cast<float>(pmn.x), static_cast<float>(pmn.y));
        mx = fmaxf(static_cast<float>(pmx.x), static_cast<float>(pmx.y));
      }
    }
    mn = wave_min(mn);
    mx = wave_max(mx);
    if constexpr (TPR > 64) {
      constexpr int NW = TPR / 64;
      float *r = red + parity * 2 * NW;  // two sets: the next row's writes cannot overtake this row's reads
      if ((tid & 63) == 0) {
        r[tid >> 6] = mn;
        r[NW + (tid >> 6)] = mx;
      }
      __syncthreads();
      mn = r[0];
      mx = r[NW];
#pragma unroll
      for (int w = 1; w < NW; ++w) {
        mn = fminf(mn, r[w]);
        mx = fmaxf(mx, r[NW + w]);
      }
    }

    RowQuant<BF16> rq;
    if constexpr (SYM) {
      rq.init_sym(static_cast<uint32_t>(mx), sym_divisor);
      if (tid == 0) meta[row] = rq.scale_bits;
    } else {
      rq.init(mn, mx, BITS);
      if (tid == 0) {
        meta[2 * row] = rq.scale_bits;
        meta[2 * row + 1] = rq.zero_bits;
      }
    }
    // ---- quantise in source order, 8 code bytes per clean group to their destination position
    auto quantise = [&](auto slow_c) {
      constexpr bool SLOW = decltype(slow_c)::value;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const uint2 c = group_codes<BITS, BF16, SLOW, SYM>(cur[i], rq);
        if ((g[i] & 0xFFu) == 0u) *reinterpret_cast<Bytes8 *>(codes_s + (g[i] >> 8)) = Bytes8{c.x, c.y};
      }
#pragma unroll
      for (int k = 0; k < ND; ++k)
        if (tid + k * TPR < ndirty) dirty_codes(dv[k], my_dirty[k], rq, slow_c);
      for (int j = tid + ND * TPR; j < ndirty; j += TPR) dirty_codes(xv[dirty_grp[j]], dirty[j], rq, slow_c);
    };
    if (__builtin_amdgcn_readfirstlane(rq.slow ? 1 : 0)) {
      quantise(std::true_type{});
    } else {
      quantise(std::false_type{});
    }
    __syncthreads();

    // ---- pack pass: 16 code bytes per lane -> 8 bytes (int4) or 16 bytes (int8)
    const int units = static_cast<int>((num_int + 15) >> 4);
    for (int u = tid; u < units; u += TPR) {
      const uint4 c = *reinterpret_cast<const uint4 *>(codes_s + u * 16);
      const int valid = static_cast<int>(num_int) - u * 16;  // codes of this unit that exist (16 except at the tail)
      if constexpr (BITS == 4) {
        // byte pairs (c0, c1) -> c0 | c1 << 4: t = w | w >> 4 leaves them in bytes 0 and 2
        const uint32_t t0 = c.x | (c.x >> 4), t1 = c.y | (c.y >> 4), t2 = c.z | (c.z >> 4), t3 = c.w | (c.w >> 4);
        const uint2 packed = make_uint2(__builtin_amdgcn_perm(t1, t0, 0x06040200u),
                                        __builtin_amdgcn_perm(t3, t2, 0x06040200u));
        uint8_t *drow = dst + row * (num_int >> 1) + u * 8;
        if (valid >= 16 && vec_out) {
          *reinterpret_cast<uint2 *>(drow) = packed;
        } else {
          for (int b = 0; b < (valid < 16 ? valid : 16) / 2; ++b)
            drow[b] = static_cast<uint8_t>((b < 4 ? packed.x : packed.y) >> (8 * (b & 3)));
        }
      } else {
        uint8_t *drow = to8 ? dst + tile8_offset(l8, row, u >> 1, u & 1) : dst + row * num_int + u * 16;
        if (valid >= 16 && vec_out) {
          *reinterpret_cast<uint4 *>(drow) = c;
        } else {
          for (int b = 0; b < (valid < 16 ? valid : 16); ++b) {
            const uint32_t w = b < 4 ? c.x : (b < 8 ? c.y : (b < 12 ? c.z : c.w));
            drow[b] = static_cast<uint8_t>(w >> (8 * (b & 3)));
          }
        }
      }
    }
  };

  // Without PF: no software prefetch; the launch makes one workgroup per row (up to the grid limit), several of
  // them are resident per CU, and their phases drift apart, so loads, arithmetic and stores of
  // different rows overlap.
  // Tile-ordered output: a cache line of the operand buffer takes pieces of 4 (heads) or 16 (tails) consecutive rows.
  // Workgroups are dealt round-robin to the 8 XCDs, so workgroup w takes row (w % 8) * rows / 8 + w / 8: rows
  // that share lines then run at about the same time on the same XCD and meet in its L2.
  const int64_t per_xcd = (rows + 7) >> 3;
  const int64_t items = to8 ? per_xcd * 8 : rows;
  int parity = 0;
  auto row_of = [&](int64_t w) -> int64_t {
    const int64_t r = to8 ? (w & 7) * per_xcd + (w >> 3) : w;
    return w < items && r < rows ? r : -1;
  };
  auto load_all = [&](int64_t row, uint4 (&v)[NV], uint4 (&dvv)[ND], uint16_t (&fv)[ND]) {
    load_row(row, v);
    const uint4 *xv = reinterpret_cast<const uint4 *>(x + row * cols);
#pragma unroll
    for (int k = 0; k < ND; ++k) {
      dvv[k] = make_uint4(0, 0, 0, 0);
      fv[k] = 0;
      if (tid + k * TPR < ndirty) dvv[k] = xv[my_dgrp[k]];
      if (tid + k * TPR < num_fp) fv[k] = x[row * cols + my_fpcol[k]];
    }
  };
  if constexpr (PF) {
    // Long rows leave room for two workgroups per CU only (registers), so the launch is persistent (a few rows per
    // workgroup) and the next row's loads are issued before the current row's arithmetic: the memory pipeline has
    // work while the workgroup reduces, quantises and stores.
    uint4 cur[NV], nxt[NV], dv[ND], dvn[ND];
    uint16_t fpv[ND], fpvn[ND];
    int64_t w = blockIdx.x;
    int64_t row = row_of(w);
    if (row >= 0) load_all(row, cur, dv, fpv);
    for (; w < items; w += gridDim.x) {
      const int64_t row2 = row_of(w + gridDim.x);
      if (row2 >= 0) load_all(row2, nxt, dvn, fpvn);
      if (row >= 0) {
        parity ^= 1;
        process(row, cur, dv, fpv, parity);
      }
#pragma unroll
      for (int i = 0; i < NV; ++i) cur[i] = nxt[i];
#pragma unroll
      for (int k = 0; k < ND; ++k) {
        dv[k] = dvn[k];
        fpv[k] = fpvn[k];
      }
      row = row2;
    }
  } else {
    for (int64_t w = blockIdx.x; w < items; w += gridDim.x) {
      const int64_t row = row_of(w);
      if (row < 0) continue;
      parity ^= 1;
      uint4 cur[NV], dv[ND];
      uint16_t fpv[ND];
      load_all(row, cur, dv, fpv);
      process(row, cur, dv, fpv, parity);
    }
  }
}

template <typename IdxT, int BITS, bool BF16>
__global__ __launch_bounds__(kThreads) void asym_quantize_kernel(
    const uint16_t *__restrict__ x, int64_t rows, int64_t cols, const IdxT *__restrict__ src_col,
    const IdxT *__restrict__ fp_col, const uint32_t *__restrict__ mask, int64_t num_int, int64_t num_fp,
    uint8_t *__restrict__ dst, uint16_t *__restrict__ meta, uint16_t *__restrict__ fp_x, int vec_ok) {
  extern __shared__ __align__(16) uint16_t row_s[];
  __shared__ float red[8];
  gather_rows<IdxT, BITS, BF16>(x, rows, cols, src_col, fp_col, mask, num_int, num_fp, dst, meta, fp_x, vec_ok, row_s,
                                red);
}

// Shapes that may stream: the column map's flag (known only on the device) picks the path.
// Dynamic LDS: the row (gather path) or one byte per code (streaming path), whichever is larger.
// SYM: symmetric activations; exists on the streaming path only (the host checks the column map's flag first).
template <typename IdxT, int BITS, bool BF16, int NV, int TPR, bool SYM = false, bool PF = false>
__global__ __launch_bounds__(TPR) void asym_quantize_stream_kernel(
    const uint16_t *__restrict__ x, int64_t rows, int64_t cols, const IdxT *__restrict__ src_col,
    const IdxT *__restrict__ fp_col, const uint32_t *__restrict__ mask, const uint32_t *__restrict__ grp,
    const uint32_t *__restrict__ dirty, const uint16_t *__restrict__ dirty_grp, const uint32_t *__restrict__ flags,
    int64_t num_int, int64_t num_fp, uint8_t *__restrict__ dst, uint16_t *__restrict__ meta,
    uint16_t *__restrict__ fp_x, int vec_out, float sym_divisor) {
  static_assert(sizeof(IdxT) == 2, "streaming needs cols <= 32768");
  extern __shared__ __align__(16) uint16_t row_s[];
  __shared__ float red[64];
  if (flags[0] & 1u) {
    uint8_t *codes_s = reinterpret_cast<uint8_t *>(row_s);
    stream_rows<BITS, BF16, NV, TPR, SYM, PF>(x, rows, cols, grp, dirty, dirty_grp, static_cast<int>(flags[1]),
                                          reinterpret_cast<const uint16_t *>(fp_col), num_int, num_fp, dst, meta, fp_x,
                                          codes_s, red, vec_out, sym_divisor);
  } else if constexpr (!SYM) {
    // Tile-ordered output exists on the streaming path only: a column map that does not stream (any other index
    // order) must not reach the row-major gather code with an operand buffer as `dst` and no `fp_x`.  Nothing is
    // written then; the entry points refuse such a column map before launching.
    if (vec_out >= 2) return;
    gather_rows<IdxT, BITS, BF16, TPR>(x, rows, cols, src_col, fp_col, mask, num_int, num_fp, dst, meta, fp_x, 1,
                                       row_s, red);
  }
}

// ---------------------------------------------------------------------------------------
// Rows of more than 8192 columns (the down_proj inputs) -> int8 operand buffer in tile order, fp16 input.
//
// One workgroup of eight waves per CU (two where two rings fit the LDS) walks over its rows; a row is copied global -> LDS with direct copies (no
// registers, so two rows are in flight while a third is worked on) into a ring of two slots.  Per row:
//   wait for this wave's copies of the row, barrier (the row is in LDS)
//   every lane reads its NV groups of 8 columns (and, lanes 0 .. ndirty-1, one group that holds outlier columns;
//   lanes 0 .. num_fp-1 one outlier value, which goes straight to the staging area); barrier (the slot is free)
//   the copies of the row after the next are issued into the slot
//   min / max, barrier, scale and zero
//   8 codes per group -> staging area in SOURCE order (one byte per column, 8 aligned bytes per group; the bytes
//   at outlier columns mean nothing), barrier
//   staging area -> operand buffer in 16-byte units: a unit takes 16 consecutive integer columns, which are 16
//   consecutive staged bytes from an offset that depends on the unit only (the outlier columns in front of it) unless
//   outlier columns lie between them; lanes 0 .. (such units) - 1 gather one of those byte by byte.  The outlier
//   values follow the codes and leave as 16-byte units as well.
// Squeezing the outlier columns out on the way OUT of the staging area keeps every LDS access aligned: 8-byte
// writes at byte offsets that are not multiples of 8 (the compacted position of a group) cost about twice the
// time of aligned ones here, and were half of this kernel's time per row.
// The arithmetic of a row takes less time than its bytes need, so the copies never wait for it; with registers as
// the prefetch target (asym_quantize_stream_kernel's persistent form) two workgroups of four waves fit a CU, a wave
// stalls in the issue of 16 loads per lane while the memory queue is full, and transfer and arithmetic add up.
// Groups past the row's end read 16 bytes of NaN kept behind the slot (min / max skip them).
constexpr int kRingThreads = 512;

// LDS bytes of the ring kernel (host and device agree through these functions)
__host__ __device__ inline int64_t ring_groups_per_lane(int64_t cols) { return (cols / 8 + kRingThreads - 1) / kRingThreads; }
__host__ __device__ inline int64_t ring_slot_bytes(int64_t cols) { return ((cols * 2 + 1023) / 1024) * 1024 + 16; }
__host__ __device__ inline int64_t ring_lds_bytes(int64_t cols, int64_t num_fp) {
  return 2 * ring_slot_bytes(cols) + ring_groups_per_lane(cols) * kRingThreads * 8 + 2 * num_fp + 32 +
         4 * (kRingThreads / 64) * sizeof(float);
}

// codes of the two halves of w in bytes 0 and 2 (int8: code = level - 128 mod 256), rows on the fast path
__device__ __forceinline__ uint32_t ring_code_pair(uint32_t w, h2 zero2, float rcp, uint32_t maxq2) {
  const uint32_t d = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, w) - zero2);
  uint32_t tb;
  asm("v_fma_mixlo_f16 %0, %1, %2, 0 op_sel_hi:[1,0,0]\n\t"
      "v_fma_mixhi_f16 %0, %1, %2, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]"
      : "=&v"(tb)
      : "v"(d), "v"(rcp));
  tb = pk_min_f16(pk_max_f16(tb, 0u), maxq2);  // NaN -> 0
  constexpr _Float16 magic = static_cast<_Float16>(1024 + 128);
  return __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, tb) + h2{magic, magic});
}

template <int NV>
__global__ __launch_bounds__(kRingThreads) void quantize_tile8_ring_kernel(
    const uint16_t *__restrict__ x, int64_t rows, int64_t cols, const uint16_t *__restrict__ fp_col,
    const uint32_t *__restrict__ grp, const uint32_t *__restrict__ dirty, const uint16_t *__restrict__ dirty_grp,
    const uint16_t *__restrict__ unit, const uint16_t *__restrict__ gather_unit,
    const uint16_t *__restrict__ gather_cols, int ndirty, int ngather, int64_t num_int, int64_t num_fp,
    uint8_t *__restrict__ dst, uint16_t *__restrict__ meta) {
  constexpr int T = kRingThreads, NW = T / 64;
  constexpr int NU = NV / 2 + 1;  // 16-byte units per lane: (codes + outlier values) / 16 / T, at most 512 outliers
  extern __shared__ __align__(16) uint8_t ring_s[];
  treat_all_nans_alike();
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nvec = static_cast<int>(cols >> 3);
  const uint32_t row_bytes = static_cast<uint32_t>(cols) * 2u;
  const uint32_t pieces = (row_bytes + 1023u) >> 10;  // direct copies move 1 KB each
  const uint32_t nan_off = pieces << 10;              // inside a slot: 16 bytes of NaN behind the row
  const uint32_t slot_stride = nan_off + 16u;
  // LDS: slot 0 | slot 1 | codes in source order (8 NV T bytes) | outlier values | 32 spare bytes (the units' second
  // 16-byte read may start there) | reduction slots
  uint8_t *codes_s = ring_s + 2 * slot_stride;
  const uint32_t fp_off = NV * T * 8;
  float *red_s = reinterpret_cast<float *>(codes_s + fp_off + 2 * num_fp + 32);  // [2][2 NW]
  const Tile8Layout l8 = tile8_layout(rows, num_int, num_fp);

  // rows of this workgroup: workgroups are dealt round-robin to the 8 XCDs and the four rows that share the cache
  // lines of the operand buffer should meet in one L2, so XCD k takes the k-th eighth of the rows
  const int64_t per_xcd = (rows + 7) >> 3, stride = gridDim.x >> 3;
  auto row_at = [&](int64_t i) -> int64_t {
    const int64_t idx = (blockIdx.x >> 3) + i * stride;
    const int64_t r = (blockIdx.x & 7) * per_xcd + idx;
    return idx < per_xcd && r < rows ? r : -1;
  };
  const uint32_t ring_lds = lds_address(ring_s);
  // copy k of this wave for a row (every wave issues NV copies per row, the count the waits below rely on: a piece
  // past the last is the last once more)
  auto issue_one = [&](int64_t row, int slot, int k) {
    const uint8_t *src = reinterpret_cast<const uint8_t *>(x + row * cols);
    const uint32_t base = ring_lds + static_cast<uint32_t>(slot) * slot_stride;
    uint32_t piece = static_cast<uint32_t>(wave + NW * k);
    piece = piece < pieces ? piece : pieces - 1u;
    uint32_t off = (piece << 10) + static_cast<uint32_t>(lane) * 16u;
    off = off < row_bytes - 16u ? off : row_bytes - 16u;  // lanes past the row's end repeat its last 16 bytes
    dma_load16(src, off, base + (piece << 10));
  };
  auto issue = [&](int64_t row, int slot) {
#pragma unroll
    for (int k = 0; k < NV; ++k) issue_one(row, slot, k);
  };

  int64_t row = row_at(0);
  if (row < 0) return;
  issue(row, 0);

  // ---- row-invariant tables of this lane, in registers
  // groups: where to read (the NaN block for groups past the row's end) and whether min / max take the group as it
  // is (a group with outlier columns is taken by one of the lanes 0 .. ndirty-1 instead, with those columns masked)
  // (every load is unconditional, from a clamped index: behind a condition each would sit in a branch of its own
  // with its own wait, one round trip to the L2 after the other)
  uint32_t gsrc[NV], keep[NV];
  uint32_t info[NV];
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int gi = tid + k * T;
    info[k] = grp[gi < nvec ? gi : nvec - 1];
  }
  const bool has_dirty = tid < ndirty, has_fp = tid < num_fp;
  // (lanes without an entry read the first words of grp, which always exist: the other tables may be empty)
  const uint16_t *spare = reinterpret_cast<const uint16_t *>(grp);
  const uint32_t d_info = *(has_dirty ? dirty + tid : grp);
  const uint32_t d_grp = *(has_dirty ? dirty_grp + tid : spare);
  const uint32_t f_col = *(has_fp ? fp_col + tid : spare);
  // units (colmap.h): consecutive columns are 16 consecutive staged bytes from the unit's first column on ("plain");
  // the others are gathered byte by byte, one unit per lane of the first `ngather` lanes
  const int nu_int = static_cast<int>(num_int >> 4), nu = nu_int + static_cast<int>(num_fp >> 3);
  uint32_t ubase[NU], ushift[NU];  // 16-byte-aligned offset into the staging area, byte shift; 0xFFFFFFFF: not plain
  uint32_t ucol[NU];
#pragma unroll
  for (int j = 0; j < NU; ++j) {
    const int u = tid + j * T;
    ucol[j] = unit[u < nu_int ? u : nu_int - 1];  // (num_int >= 64: at least four units)
  }
  const bool has_gather = tid < ngather;
  uint32_t goff[8];  // staged byte offsets (= columns) of the 16 codes of this lane's gathered unit, two per register
  const int gunit = *(has_gather ? gather_unit + tid : spare);
  {
    const uint4 *c = reinterpret_cast<const uint4 *>(has_gather ? gather_cols + 16 * tid : spare);
    const uint4 a = c[0], b = c[1];
    goff[0] = a.x, goff[1] = a.y, goff[2] = a.z, goff[3] = a.w;
    goff[4] = b.x, goff[5] = b.y, goff[6] = b.z, goff[7] = b.w;
  }
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int gi = tid + k * T;
    gsrc[k] = gi < nvec ? static_cast<uint32_t>(gi) * 16u : nan_off;
    keep[k] = gi >= nvec || (info[k] & 0xFFu) == 0u ? 0xFFFFFFFFu : 0u;
  }
  const uint32_t d_mask = has_dirty ? d_info & 0xFFu : 0xFFu;
  const uint32_t d_src = has_dirty ? d_grp * 16u : nan_off;
  const uint32_t f_src = has_fp ? f_col * 2u : 0u;
#pragma unroll
  for (int j = 0; j < NU; ++j) {
    const int u = tid + j * T;
    uint32_t off = 0xFFFFFFFFu;
    if (u < nu_int) {
      if (ucol[j] != 0xFFFFu) off = ucol[j];
    } else if (u < nu) {
      off = fp_off + static_cast<uint32_t>(u - nu_int) * 16u;
    }
    ubase[j] = off == 0xFFFFFFFFu ? off : off & ~15u;
    ushift[j] = off & 15u;
  }
  if (tid < 4) {
    reinterpret_cast<uint32_t *>(ring_s + nan_off)[tid] = 0xFFFFFFFFu;
    reinterpret_cast<uint32_t *>(ring_s + slot_stride + nan_off)[tid] = 0xFFFFFFFFu;
  }
  // the tables are complete here (this also waits for the first row), not at their first use inside the loop,
  // where a wait for them would wait for the copies in flight as well
#pragma unroll
  for (int k = 0; k < NV; ++k) asm volatile("" ::"v"(gsrc[k]), "v"(keep[k]));
#pragma unroll
  for (int j = 0; j < NU; ++j) asm volatile("" ::"v"(ubase[j]), "v"(ushift[j]));
#pragma unroll
  for (int j = 0; j < 8; ++j) asm volatile("" ::"v"(goff[j]));
  asm volatile("" ::"v"(d_mask), "v"(d_src), "v"(f_src), "v"(gunit));
  {
    const int64_t r1 = row_at(1);
    if (r1 >= 0) issue(r1, 1);
  }

  const uint32_t maxq2 = 0x5BF85BF8u;  // 255.0 in both halves
  for (int64_t i = 0; row >= 0; ++i) {
    const int slot = static_cast<int>(i & 1);
    const int64_t row1 = row_at(i + 1), row2 = row_at(i + 2);
    // This wave's copies of the row have landed.  Memory operations complete in the order of their issue; the NV
    // newest at this point are stores of the last row and, before them, copies of the next row, so "at most NV
    // outstanding" covers the NV copies of this row, which are older than all of those.
    if (row1 >= 0) {
      __builtin_amdgcn_s_waitcnt(vmcnt_imm(NV));
    } else {
      __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    }
    __syncthreads();
    const uint8_t *slot_s = ring_s + static_cast<uint32_t>(slot) * slot_stride;
    uint4 v[NV];
#pragma unroll
    for (int k = 0; k < NV; ++k) v[k] = *reinterpret_cast<const uint4 *>(slot_s + gsrc[k]);
    const uint4 dv = *reinterpret_cast<const uint4 *>(slot_s + d_src);
    const uint16_t fpv = *reinterpret_cast<const uint16_t *>(slot_s + f_src);
    // (the staging area is free: every wave has finished the last row's stores before the barrier above)
    if (has_fp) reinterpret_cast<uint16_t *>(codes_s + fp_off)[tid] = fpv;
    __syncthreads();

    // ---- min / max; the copies of the row after the next go out between the groups (the address unit takes a
    // copy every 16 cycles: issued in one run, the eight waves would queue behind each other for half a microsecond)
    uint32_t pmn_b = 0x7C007C00u, pmx_b = 0xFC00FC00u;  // +inf / -inf in both halves
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      if (row2 >= 0) issue_one(row2, slot, k);
      const uint32_t lo = pk_min_f16(pk_min_f16(v[k].x, v[k].y), pk_min_f16(v[k].z, v[k].w));
      const uint32_t hi = pk_max_f16(pk_max_f16(v[k].x, v[k].y), pk_max_f16(v[k].z, v[k].w));
      pmn_b = pk_min_f16(pmn_b, (lo & keep[k]) | (0x7C007C00u & ~keep[k]));
      pmx_b = pk_max_f16(pmx_b, (hi & keep[k]) | (0xFC00FC00u & ~keep[k]));
    }
    if (has_dirty) {
      // outlier halves become 0xFFFF, a quiet NaN, which min / max skip
      const uint32_t w[4] = {dv.x, dv.y, dv.z, dv.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_sbfe(static_cast<int>(d_mask), 2 * k, 1));
        const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_sbfe(static_cast<int>(d_mask), 2 * k + 1, 1));
        const uint32_t m = w[k] | __builtin_amdgcn_perm(hi, lo, 0x07060100u);
        pmn_b = pk_min_f16(pmn_b, m);
        pmx_b = pk_max_f16(pmx_b, m);
      }
    }
    const h2 pmn = __builtin_bit_cast(h2, pmn_b), pmx = __builtin_bit_cast(h2, pmx_b);
    float mn = fminf(static_cast<float>(pmn.x), static_cast<float>(pmn.y));
    float mx = fmaxf(static_cast<float>(pmx.x), static_cast<float>(pmx.y));
    mn = wave_min(mn);
    mx = wave_max(mx);
    float *r = red_s + slot * 2 * NW;  // two sets: the next row's writes cannot overtake this row's reads
    if (lane == 0) {
      r[wave] = mn;
      r[NW + wave] = mx;
    }
    __syncthreads();
    mn = r[0];
    mx = r[NW];
#pragma unroll
    for (int w = 1; w < NW; ++w) {
      mn = fminf(mn, r[w]);
      mx = fmaxf(mx, r[NW + w]);
    }
    RowQuant<false> rq;
    rq.init(mn, mx, 8);
    if (tid == 0) {
      meta[2 * row] = rq.scale_bits;
      meta[2 * row + 1] = rq.zero_bits;
    }

    // ---- codes -> staging area, source order
    uint2 *stage8 = reinterpret_cast<uint2 *>(codes_s) + tid;
    if (__builtin_amdgcn_readfirstlane(rq.slow ? 1 : 0)) {
#pragma unroll
      for (int k = 0; k < NV; ++k) stage8[k * T] = group_codes<8, false, true>(v[k], rq);
    } else {
      const _Float16 zh = static_cast<_Float16>(rq.zero);
      const h2 zero2 = h2{zh, zh};
#pragma unroll
      for (int k = 0; k < NV; ++k) {
        const uint32_t p0 = ring_code_pair(v[k].x, zero2, rq.rcp, maxq2), p1 = ring_code_pair(v[k].y, zero2, rq.rcp, maxq2);
        const uint32_t p2 = ring_code_pair(v[k].z, zero2, rq.rcp, maxq2), p3 = ring_code_pair(v[k].w, zero2, rq.rcp, maxq2);
        stage8[k * T] = make_uint2(__builtin_amdgcn_perm(p1, p0, 0x06040200u), __builtin_amdgcn_perm(p3, p2, 0x06040200u));
      }
    }
    __syncthreads();

    // ---- staging area -> operand buffer, 16 bytes per lane and unit
    // chunk (step, h) of the row is at + 2048 step + 16 (h ^ bit 3 of the row) from here (tile8_offset)
    uint8_t *drow = dst + (row >> 6) * l8.block_bytes + ((row >> 5) & 1) * 1024 + (row & 31) * 32;
    const uint32_t swap16 = static_cast<uint32_t>((row >> 3) & 1) << 4;
    auto unit_at = [&](int u) -> uint4 * {
      return reinterpret_cast<uint4 *>(drow + ((static_cast<uint32_t>(u >> 1) << 11) | ((static_cast<uint32_t>(u & 1) << 4) ^ swap16)));
    };
#pragma unroll
    for (int j = 0; j < NU; ++j) {
      if (ubase[j] != 0xFFFFFFFFu) {
        // 16 bytes from byte offset ubase + ushift: two aligned 16-byte reads, then a shift by whole words (two
        // levels of selects) and by bytes
        const uint4 a = *reinterpret_cast<const uint4 *>(codes_s + ubase[j]);
        const uint4 b = *reinterpret_cast<const uint4 *>(codes_s + ubase[j] + 16);
        uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
        // (selects written as bit masks: as conditional moves between array elements the compiler turns them into
        // one dynamically indexed array in scratch memory, whose loads would wait for the copies in flight)
        const uint32_t by2 = 0u - ((ushift[j] >> 3) & 1u), by1 = 0u - ((ushift[j] >> 2) & 1u);
#pragma unroll
        for (int t = 0; t < 6; ++t) w[t] = (w[t + 2] & by2) | (w[t] & ~by2);
#pragma unroll
        for (int t = 0; t < 5; ++t) w[t] = (w[t + 1] & by1) | (w[t] & ~by1);
        uint4 c;
        c.x = __builtin_amdgcn_alignbyte(w[1], w[0], ushift[j]);
        c.y = __builtin_amdgcn_alignbyte(w[2], w[1], ushift[j]);
        c.z = __builtin_amdgcn_alignbyte(w[3], w[2], ushift[j]);
        c.w = __builtin_amdgcn_alignbyte(w[4], w[3], ushift[j]);
        *unit_at(tid + j * T) = c;
      }
    }
    if (has_gather) {
      uint32_t c[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const uint32_t b0 = codes_s[goff[2 * t] & 0xFFFFu], b1 = codes_s[goff[2 * t] >> 16];
        const uint32_t b2 = codes_s[goff[2 * t + 1] & 0xFFFFu], b3 = codes_s[goff[2 * t + 1] >> 16];
        c[t] = b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
      }
      *unit_at(gunit) = make_uint4(c[0], c[1], c[2], c[3]);
    }
    row = row1;
  }
}

// 4-bit LEVELS (code + 8, 0 .. 15) of the two fp16 halves of w in bytes 0 and 2 of the result, for rows on the fast
// path (finite range, scale >= 1e-6; RowQuant::slow == false); same levels as code_pair gives.
//   asymmetric: d = fp16(x - zero); t = fp16(f32(d) * rcp); t = max(t, 0) (a NaN element becomes 0, as the
//   reference's integer conversion makes it); t + 1024 holds rne(t) in its low mantissa bits.  No upper clamp:
//   on this path t < 15.5 for every fp16 scale (x - zero <= max - min, the scale is at least fp16((max - min) / 15),
//   and over all fp16 scales >= 1e-6 the largest quotient, reached at the smallest, subnormal scale, is 15.47;
//   tests/test_quotient_levels.py enumerates them).
//   symmetric: t = fp16(f32(x) * rcp) with |t| <= 4.2 (scale = fp16(max|x| / 4), at most 3 % below the quotient
//   for the smallest scale); t + 1544 holds rne(t) + 8 in its low mantissa bits.
// (The two v_fma_mix instructions write the low and the high half of one register: the output is early-clobber
// because the second one still reads the inputs after the first has written; VALU to VALU, no wait states needed.)
template <bool SYM, class RQ>
__device__ __forceinline__ uint32_t level_pair_fast(uint32_t w, const RQ &rq) {
  uint32_t d = w, tb;
  if constexpr (!SYM) {
    const _Float16 zh = static_cast<_Float16>(rq.zero);
    d = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, w) - h2{zh, zh});
  }
  asm("v_fma_mixlo_f16 %0, %1, %2, 0 op_sel_hi:[1,0,0]\n\t"
      "v_fma_mixhi_f16 %0, %1, %2, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]"
      : "=&v"(tb)
      : "v"(d), "v"(rq.rcp));
  if constexpr (!SYM) tb = pk_max_f16(tb, 0u);
  constexpr _Float16 magic = static_cast<_Float16>(SYM ? 1544 : 1024);
  return __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, tb) + h2{magic, magic});
}

// ---------------------------------------------------------------------------------------
// 6-bit operand buffers (consumer: gemm_fp6.h), written in the in-place order of the column map.
//
// One wave per row.  The wave copies the row global -> LDS with 16-byte-per-lane direct copies (no
// registers are held while the row is in flight).  A copy instruction moves one contiguous kilobyte
// (64 groups of 8 columns = 16 fragments of 32 consecutive source columns; whole cache lines) and deals
// it to the LDS slots transposed: slot 16 i + m of the kilobyte holds group 4 m + i, i.e. the i-th group
// of the kilobyte's fragment m.  Lane L owns the fragments L, L + 64, ...; its i-th 16-byte read of a
// fragment and those of its 15 neighbours cover 256 consecutive bytes, so all reads are free of bank
// conflicts.  In the image the holes (outlier columns among the first num_int columns) are
// overwritten with their fillers (integer columns of the tail), two-byte LDS copies with row-invariant
// addresses held in registers; after that the first num_int columns ARE the integer operand, in place:
// one pass over the image for min / max, a second one that turns each fragment into 32 levels, packs
// them to 24 bytes in registers and stores head and tail.  No barrier, no cross-wave reduction (a wave's
// LDS operations execute in order), no data moved between lanes except the two reductions.
// A workgroup (= wave) walks over rows w, w + grid, ...; up to eight of them share a CU (two per SIMD),
// so one wave's arithmetic covers the other's transfer and LDS waits.  JT > 0: fragments per lane known at
// compile time (rows up to 10240 columns); 0: a run-time loop over them.
template <bool BF16, bool SYM, int JT, int W>
__global__ __launch_bounds__(64 * W) void quantize_fp6_wave_kernel(
    const uint16_t *__restrict__ x, int64_t rows, int cols, const uint32_t *__restrict__ patch,
    const uint16_t *__restrict__ fp_col, int nholes, int num_int, int num_fp,
    uint8_t *__restrict__ dst, uint16_t *__restrict__ meta, float sym_divisor) {
  static_assert(!(BF16 && SYM), "symmetric activations are fp16");
  constexpr int kTogether = 2;  // waves that issue their copies at the same time (measured: 1, 2, 4 and all 8)
  extern __shared__ __align__(16) uint8_t images[];
  __shared__ int turn_s;
  if constexpr (!BF16 && !SYM) treat_all_nans_alike();  // pass 1 uses pk_min_f16 / pk_max_f16 on the raw row
  // (nholes: the column map's count of holes, which the host knows: the entry points look the map's flag words up
  // before launching, and refuse a map without the in-place order; the kernel starts without a dependent load)
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  const int frags_all = cols >> 5, frags = num_int >> 5, nchunk = num_fp >> 3;
  const int J = JT > 0 ? JT : (frags_all + 63) >> 6;
  uint8_t *row_img = images + wave * (J * 4096);
  if (threadIdx.x == 0) turn_s = 0;
  __syncthreads();
  const Fp6Layout l6 = fp6_layout(rows, num_int, num_fp);
  const uint32_t lds0 = lds_address(row_img);

  constexpr int PREG = 4;
  uint32_t p_hole[PREG], p_fill[PREG], o_addr[8];
  // byte offset of source column c inside a row image
  auto img_of_col = [](uint32_t c) -> uint32_t {
    const uint32_t g = c >> 3, f = g >> 2, i = g & 3u;
    return ((f >> 4) << 10) + ((16u * i + (f & 15u)) << 4) + ((c & 7u) << 1);
  };
  // body(j) for this lane's fragment slots j = 0 .. J-1, unrolled when their number is known at compile time
  auto for_j = [&](auto body) {
    if constexpr (JT > 0) {
#pragma unroll
      for (int j = 0; j < JT; ++j) body(j);
    } else {
      for (int j = 0; j < J; ++j) body(j);
    }
  };
  auto issue = [&](int64_t row) {
    const uint64_t a = reinterpret_cast<uint64_t>(x + row * cols);
    // (the intrinsic returns int: each half goes through uint32_t, or the low half would be sign-extended)
    const uint32_t a_hi = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(a >> 32)));
    const uint32_t a_lo = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(a & 0xFFFFFFFFu)));
    const uint8_t *rp = reinterpret_cast<const uint8_t *>((static_cast<uint64_t>(a_hi) << 32) | a_lo);
    // kilobyte q of the row: this lane copies group 64 q + 4 (lane % 16) + lane / 16 to slot 64 q + lane.
    // The kilobytes are requested in an order that starts at a row-dependent one and wraps around: all waves of
    // the launch issue their copies at about the same time, and with every row starting at its kilobyte 0 (rows
    // are a multiple of 1 KB apart) the requests in flight at any moment would share their low address bits and
    // crowd onto a few memory channels (measured with the input in HBM: 15.8 -> 14.0 us for 2048 x 8192).
    const int g_in = 4 * (lane & 15) + (lane >> 4), g_last = (cols >> 3) - 1;
    const int nkb = 4 * J;
    const int rot = __builtin_amdgcn_readfirstlane(static_cast<int>((row * 5) % nkb));
    for_j([&](int j) {
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        int q = 4 * j + t + rot;
        q = q >= nkb ? q - nkb : q;
        const int g = 64 * q + g_in;
        const uint32_t voff = static_cast<uint32_t>(g < g_last ? g : g_last) * 16u;  // past the row: any valid group
        dma_load16(rp, voff, lds0 + q * 1024);
      }
    });
  };

  auto process = [&](int64_t row, uint8_t *img) {
    auto ld16 = [&](uint32_t off) { return *reinterpret_cast<const uint16_t *>(img + off); };
    // ---- outlier values, 8 per lane, to the outlier units of the operand buffer (before the holes are patched:
    // holes are outlier columns)
    if (lane < nchunk) {
      uint4 o;
      o.x = ld16(o_addr[0]) | (static_cast<uint32_t>(ld16(o_addr[1])) << 16);
      o.y = ld16(o_addr[2]) | (static_cast<uint32_t>(ld16(o_addr[3])) << 16);
      o.z = ld16(o_addr[4]) | (static_cast<uint32_t>(ld16(o_addr[5])) << 16);
      o.w = ld16(o_addr[6]) | (static_cast<uint32_t>(ld16(o_addr[7])) << 16);
      *reinterpret_cast<uint4 *>(dst + fp6_outlier_offset(l6, row, lane >> 1, lane & 1)) = o;
    }
    for (int c = lane + 64; c < nchunk; c += 64) {
      uint32_t w[4];
#pragma unroll
      for (int k = 0; k < 4; ++k)
        w[k] = ld16(img_of_col(fp_col[c * 8 + 2 * k])) |
               (static_cast<uint32_t>(ld16(img_of_col(fp_col[c * 8 + 2 * k + 1]))) << 16);
      *reinterpret_cast<uint4 *>(dst + fp6_outlier_offset(l6, row, c >> 1, c & 1)) = make_uint4(w[0], w[1], w[2], w[3]);
    }
    // ---- holes <- fillers
#pragma unroll
    for (int k = 0; k < PREG; ++k)
      if (lane + 64 * k < nholes) *reinterpret_cast<uint16_t *>(img + p_hole[k]) = ld16(p_fill[k]);
    for (int e = lane + 64 * PREG; e < nholes; e += 64) {
      const uint32_t pe = patch[e];
      *reinterpret_cast<uint16_t *>(img + img_of_col(pe & 0xFFFFu)) = ld16(img_of_col(pe >> 16));
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // other lanes read the patched halves below
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    auto load_fragment = [&](int j, uint4 (&v)[4]) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        v[i] = *reinterpret_cast<const uint4 *>(img + ((4 * j + (lane >> 4)) << 10) + ((16 * i + (lane & 15)) << 4));
    };
    // ---- pass 1: min / max (symmetric: largest |x| pattern) over this lane's fragments
    const float inf = __builtin_inff();
    float mn = inf, mx = -inf;
    uint32_t pmn_b = 0x7C007C00u, pmx_b = 0xFC00FC00u;  // +inf / -inf in both halves
    u2 amax = u2{0, 0};
    // up to four fragments per lane stay in registers from the first pass to the second (64 registers): the second
    // pass then has no LDS round trip in front of its arithmetic
    constexpr bool kKeep = JT > 0 && JT <= 4;
    uint4 kept[kKeep ? JT : 1][4];
    for_j([&](int j) {
      if (lane + 64 * j < frags) {
        uint4 v[4];
        load_fragment(j, v);
        if constexpr (kKeep) {
#pragma unroll
          for (int i = 0; i < 4; ++i) kept[j][i] = v[i];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t w[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
          if constexpr (SYM) {
#pragma unroll
            for (int k = 0; k < 4; ++k) amax = __builtin_elementwise_max(amax, __builtin_bit_cast(u2, w[k] & 0x7FFF7FFFu));
          } else if constexpr (!BF16) {
            // packed fp16 min / max skip NaN operands, as the reference's __hmin / __hmax do
            const uint32_t lo = pk_min_f16(pk_min_f16(w[0], w[1]), pk_min_f16(w[2], w[3]));
            const uint32_t hi = pk_max_f16(pk_max_f16(w[0], w[1]), pk_max_f16(w[2], w[3]));
            pmn_b = pk_min_f16(pmn_b, lo);
            pmx_b = pk_max_f16(pmx_b, hi);
          } else {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              const float f0 = __uint_as_float(w[k] << 16), f1 = __uint_as_float(w[k] & 0xFFFF0000u);
              mn = fminf(mn, fminf(f0, f1));
              mx = fmaxf(mx, fmaxf(f0, f1));
            }
          }
        }
      }
    });
    const h2 pmn = __builtin_bit_cast(h2, pmn_b), pmx = __builtin_bit_cast(h2, pmx_b);
    if constexpr (SYM) {
      mn = 0.0f;
      mx = static_cast<float>(amax.x > amax.y ? amax.x : amax.y);  // a 15-bit integer: exact, ordered like the patterns
    } else if constexpr (!BF16) {
      mn = fminf(static_cast<float>(pmn.x), static_cast<float>(pmn.y));
      mx = fmaxf(static_cast<float>(pmx.x), static_cast<float>(pmx.y));
    }
    mn = wave_min(mn);
    mx = wave_max(mx);
    RowQuant<BF16> rq;
    if constexpr (SYM) {
      rq.init_sym(static_cast<uint32_t>(mx), sym_divisor);
      if (lane == 0) meta[row] = rq.scale_bits;
    } else {
      rq.init(mn, mx, 4);
      if (lane == 0) {
        meta[2 * row] = rq.scale_bits;
        meta[2 * row + 1] = rq.zero_bits;
      }
    }
    // ---- pass 2: fragment -> 32 levels -> 24 bytes
    // (store addresses: the row's part is wave-uniform, the fragment's part is the unit 3072 (f / 2) and its half)
    const int64_t rb = (row >> 6) * l6.block_bytes;
    uint8_t *head_row = dst + rb + ((row >> 5) & 1) * 1024 + (row & 31) * 32;
    uint8_t *tail_row = dst + rb + 2048 + (row & 63) * 8;
    const uint32_t swap16 = static_cast<uint32_t>((row >> 3) & 1) << 4;
    int sum = 0;
    auto quantise = [&](auto slow_c) {
      constexpr bool SLOW = decltype(slow_c)::value;
      for_j([&](int j) {
        const int f = lane + 64 * j;
        if (f < frags) {
          uint4 v[4];
          if constexpr (kKeep) {
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = kept[j][i];
          } else {
            load_fragment(j, v);
          }
          uint32_t b[8];  // 32 levels, one per byte
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            if constexpr (!SLOW && !BF16) {
              const uint32_t p0 = level_pair_fast<SYM>(v[i].x, rq), p1 = level_pair_fast<SYM>(v[i].y, rq);
              const uint32_t p2 = level_pair_fast<SYM>(v[i].z, rq), p3 = level_pair_fast<SYM>(v[i].w, rq);
              b[2 * i] = __builtin_amdgcn_perm(p1, p0, 0x06040200u);  // bytes 0, 2 of p0 then bytes 0, 2 of p1
              b[2 * i + 1] = __builtin_amdgcn_perm(p3, p2, 0x06040200u);
            } else {
              const uint2 c = group_codes<4, BF16, SLOW, SYM>(v[i], rq);  // code nibbles (two's complement), one per byte
              b[2 * i] = c.x ^ 0x08080808u;                               // level = code + 8
              b[2 * i + 1] = c.y ^ 0x08080808u;
            }
          }
#pragma unroll
          for (int i = 0; i < 8; ++i) sum = __builtin_amdgcn_udot4(b[i], 0x01010101u, sum, false);
          uint32_t o[6];
          fp6_pack_fragment(b, o);
          const uint32_t unit = static_cast<uint32_t>(f >> 1) * 3072u, h = static_cast<uint32_t>(f & 1);
          // (default cache policy: a 128-byte line of the operand buffer takes pieces of 4 (heads) or 16 (tails) rows,
          // which meet in the XCD's L2; as streaming stores every piece went to memory on its own and the launch
          // took 29 us instead of 12)
          *reinterpret_cast<uint4 *>(head_row + unit + ((h << 4) ^ swap16)) = make_uint4(o[0], o[1], o[2], o[3]);
          *reinterpret_cast<uint2 *>(tail_row + unit + h * 512u) = make_uint2(o[4], o[5]);
        }
      });
    };
    if (__builtin_amdgcn_readfirstlane(rq.slow ? 1 : 0)) {
      quantise(std::true_type{});
    } else {
      quantise(std::false_type{});
    }
    sum = wave_sum(sum);
    if (lane == 0) reinterpret_cast<int32_t *>(dst + l6.sums_off)[row] = sum;
  };

  // Workgroup g takes the rows (g % 8) * rows / 8 + (g / 8) * W + wave (a cache line of the operand buffer takes
  // pieces of 4 (heads) or 16 (tails) consecutive rows; workgroups are dealt round-robin to the 8 XCDs, so rows that
  // share lines run on the same XCD at about the same time and meet in its L2), then every gridDim.x-th further group.
  //
  // The waves of a workgroup issue their copies kTogether at a time, in the order of a counter in LDS: the memory
  // system serves a CU's requests about in the order they arrive, so the rows land in that order and a wave does
  // its arithmetic while the later rows are still in flight.  (With all waves issuing at once the requests
  // interleave, all rows land together at the end of the transfer, and transfer and arithmetic add up instead of
  // overlapping.)  Every wave takes every one of its turns, with or without a row, so the counter always advances.
  const int64_t per_xcd = (rows + 7) >> 3, groups_per_xcd = (per_xcd + W - 1) / W, groups = groups_per_xcd * 8;
  auto row_of = [&](int64_t g) -> int64_t {
    const int64_t i = (g >> 3) * W + wave;
    const int64_t r = (g & 7) * per_xcd + i;
    return i < per_xcd && r < rows ? r : -1;
  };
  volatile int *turn_v = &turn_s;
  auto take_turn = [&](int t, int64_t row) {
    const int need = t / kTogether * kTogether;  // all waves of the earlier sets have issued
    while (__builtin_amdgcn_readfirstlane(*turn_v) < need) __builtin_amdgcn_s_sleep(1);
    if (row >= 0) issue(row);
    if (lane == 0) __hip_atomic_fetch_add(&turn_s, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  };
  int64_t g = blockIdx.x;
  if (g >= groups) return;
  int t = wave;
  take_turn(t, row_of(g));
  // Row-invariant addresses in registers: this lane's first four patches and its first chunk of 8 outliers.  The
  // loads are unconditional (clamped indices, one 16-byte load for the eight outlier columns) and come after the
  // first row's copies, so they are all in flight together and behind the row, not in front of it.
  {
    const int last_hole = nholes > 0 ? nholes - 1 : 0;
    uint32_t e[PREG];
#pragma unroll
    for (int k = 0; k < PREG; ++k) e[k] = patch[lane + 64 * k < nholes ? lane + 64 * k : last_hole];
    const int chunk = lane < nchunk ? lane : 0;
    const uint4 oc = nchunk > 0 ? *reinterpret_cast<const uint4 *>(fp_col + chunk * 8) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int k = 0; k < PREG; ++k) {
      p_hole[k] = img_of_col(e[k] & 0xFFFFu);
      p_fill[k] = img_of_col(e[k] >> 16);
    }
    const uint32_t ow[4] = {oc.x, oc.y, oc.z, oc.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      o_addr[2 * k] = img_of_col(ow[k] & 0xFFFFu);
      o_addr[2 * k + 1] = img_of_col(ow[k] >> 16);
    }
  }
  for (; g < groups; g += gridDim.x) {
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));  // this row's image has landed
    const int64_t row = row_of(g);
    if (row >= 0) process(row, row_img);
    if (g + gridDim.x < groups) {
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // this row's LDS reads are done before the image is overwritten (a wait only: no hazard)
      t += W;
      take_turn(t, row_of(g + gridDim.x));
    }
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

template <typename IdxT, int BITS, bool BF16, int NV, int TPR, bool SYM = false, bool PF = false>
int launch_stream(const void *x, int64_t rows, int64_t cols, const uint8_t *cm, const ColmapLayout &l, int64_t num_int,
                  int64_t num_fp, void *dst, void *meta, void *fp_x, hipStream_t st, bool tiled,
                  float sym_divisor = 1.0f) {
  auto kern = asym_quantize_stream_kernel<IdxT, BITS, BF16, NV, TPR, SYM, PF>;
  // the row (gather path) or one byte per code (streaming path); a tile-ordered launch only ever streams
  const int64_t lds = tiled ? align16(num_int) : align16(cols * 2);
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    if (e != hipSuccess) {
      set_last_hip_error(e);
      return QUIK_ERR_LAUNCH;
    }
  }
  const int64_t items = tiled ? (rows + 7) / 8 * 8 : rows;
  int grid = static_cast<int>(items < (int64_t(1) << 30) ? items : (int64_t(1) << 30));
  if (PF && grid > 2 * num_cus()) grid = 2 * num_cus();  // persistent: the workgroups that are resident at once
  // tiled: dst is an operand buffer in tile order (6-bit levels for 4 bits, int8 for 8 bits)
  const int vec_out = tiled ? (BITS == 4 ? 2 : 3) : (num_int % 16 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(TPR), static_cast<size_t>(lds), st,
                     static_cast<const uint16_t *>(x), rows, cols, reinterpret_cast<const IdxT *>(cm),
                     reinterpret_cast<const IdxT *>(cm + l.off_fp), reinterpret_cast<const uint32_t *>(cm + l.off_mask),
                     reinterpret_cast<const uint32_t *>(cm + l.off_grp),
                     reinterpret_cast<const uint32_t *>(cm + l.off_dirty),
                     reinterpret_cast<const uint16_t *>(cm + l.off_slot),
                     reinterpret_cast<const uint32_t *>(cm + l.off_flags), num_int, num_fp,
                     static_cast<uint8_t *>(dst), static_cast<uint16_t *>(meta), static_cast<uint16_t *>(fp_x), vec_out,
                     sym_divisor);
  return check_launch();
}

// symmetric activations through the streaming kernel (fp16; the caller has checked that the column map streams)
template <int BITS>
int launch_sym_stream(const void *x, int64_t rows, int64_t cols, const uint8_t *cm, const ColmapLayout &l,
                      int64_t num_int, int64_t num_fp, void *dst, void *scale, void *fp_x, hipStream_t st, bool tiled,
                      float divisor) {
  const int64_t groups = cols / 8;
#define QUIK_SYM_STREAM(NV)                                                                                       \
  return launch_stream<uint16_t, BITS, false, NV, kThreads, true>(x, rows, cols, cm, l, num_int, num_fp, dst, scale, \
                                                                  fp_x, st, tiled, divisor)
  if (groups <= 512) QUIK_SYM_STREAM(2);
  if (groups <= 1024) QUIK_SYM_STREAM(4);
  if (groups <= 2048) QUIK_SYM_STREAM(8);
  QUIK_SYM_STREAM(16);
#undef QUIK_SYM_STREAM
}

// Long fp16 rows -> int8 operand buffer through the LDS ring (quantize_tile8_ring_kernel).  `ndirty`: groups of 8
// columns that hold outlier columns, from the host's copy of the column map's flag words.
constexpr int64_t kLdsPerCu = 160 * 1024;
// rows of more than 8192 columns: measured against the streaming kernel at 2048 rows, kernel time from a cold
// cache: 8192 columns 17.4 against 16.8 us, 11008 19.9 against 20.9, 13824 23.7 against 26.3, 28672 41.6 against 51.0
constexpr int64_t kRingMinGroups = 2 * kRingThreads + 1;
bool ring_fits(int64_t cols, int64_t num_int, int64_t num_fp, int64_t ndirty) {
  const int64_t groups = cols / 8;
  return groups >= kRingMinGroups && groups <= 8 * kRingThreads && ndirty >= 0 && ndirty <= kRingThreads &&
         num_fp <= kRingThreads && num_int % 16 == 0 && ring_lds_bytes(cols, num_fp) <= kLdsPerCu;
}
template <int NV>
int launch_tile8_ring_nv(const void *x, int64_t rows, int64_t cols, const uint8_t *cm, const ColmapLayout &l,
                         int64_t num_int, int64_t num_fp, int ndirty, int ngather, void *dst, void *meta,
                         hipStream_t st) {
  auto kern = quantize_tile8_ring_kernel<NV>;
  const int64_t lds = ring_lds_bytes(cols, num_fp);
  if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
      e != hipSuccess) {
    set_last_hip_error(e);
    return QUIK_ERR_LAUNCH;
  }
  const int64_t per_xcd = (rows + 7) / 8;
  // one workgroup per CU when the ring takes most of its LDS, two when two fit; a multiple of the XCDs
  int64_t grid = num_cus() / 8 * 8 * (2 * lds + 1024 <= kLdsPerCu ? 2 : 1);
  if (grid < 8) grid = 8;
  if (grid > per_xcd * 8) grid = per_xcd * 8;
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(grid)), dim3(kRingThreads), static_cast<size_t>(lds), st,
                     static_cast<const uint16_t *>(x), rows, cols, reinterpret_cast<const uint16_t *>(cm + l.off_fp),
                     reinterpret_cast<const uint32_t *>(cm + l.off_grp),
                     reinterpret_cast<const uint32_t *>(cm + l.off_dirty),
                     reinterpret_cast<const uint16_t *>(cm + l.off_slot),
                     reinterpret_cast<const uint16_t *>(cm + l.off_unit),
                     reinterpret_cast<const uint16_t *>(cm + l.off_gunit),
                     reinterpret_cast<const uint16_t *>(cm + l.off_gcols), ndirty, ngather, num_int, num_fp,
                     static_cast<uint8_t *>(dst), static_cast<uint16_t *>(meta));
  return check_launch();
}
int launch_tile8_ring(const void *x, int64_t rows, int64_t cols, const uint8_t *cm, const ColmapLayout &l,
                      int64_t num_int, int64_t num_fp, int ndirty, int ngather, void *dst, void *meta,
                      hipStream_t st) {
  switch ((cols / 8 + kRingThreads - 1) / kRingThreads) {
    case 3: return launch_tile8_ring_nv<3>(x, rows, cols, cm, l, num_int, num_fp, ndirty, ngather, dst, meta, st);
    case 4: return launch_tile8_ring_nv<4>(x, rows, cols, cm, l, num_int, num_fp, ndirty, ngather, dst, meta, st);
    case 5: return launch_tile8_ring_nv<5>(x, rows, cols, cm, l, num_int, num_fp, ndirty, ngather, dst, meta, st);
    case 6: return launch_tile8_ring_nv<6>(x, rows, cols, cm, l, num_int, num_fp, ndirty, ngather, dst, meta, st);
    case 7: return launch_tile8_ring_nv<7>(x, rows, cols, cm, l, num_int, num_fp, ndirty, ngather, dst, meta, st);
    default: return launch_tile8_ring_nv<8>(x, rows, cols, cm, l, num_int, num_fp, ndirty, ngather, dst, meta, st);
  }
}

template <typename IdxT, int BITS, bool BF16>
int launch_asym(const void *x, int64_t rows, int64_t cols, const uint8_t *cm, const ColmapLayout &l, int64_t num_int,
                int64_t num_fp, void *dst, void *meta, void *fp_x, hipStream_t st, bool tiled = false,
                int64_t ndirty = -1, int64_t ngather = 0) {
  const IdxT *src_col = reinterpret_cast<const IdxT *>(cm);
  const IdxT *fp_col = reinterpret_cast<const IdxT *>(cm + l.off_fp);
  const uint32_t *mask = reinterpret_cast<const uint32_t *>(cm + l.off_mask);
  if constexpr (sizeof(IdxT) == 2) if (cols <= kStreamMaxCols && cols % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0) {
    // Four waves per row, one row per workgroup: more, shorter waves hide the load and LDS latencies
    // better than fewer waves with less per-row fixed work (measured with 64, 128 and 256 threads).
    const int64_t groups = cols / 8;
#define QUIK_STREAM(NV) \
  return launch_stream<IdxT, BITS, BF16, NV, kThreads>(x, rows, cols, cm, l, num_int, num_fp, dst, meta, fp_x, st, tiled)
    // fp16 rows beyond 8192 columns with tile-ordered int8 output: the LDS ring kernel
    if constexpr (BITS == 8 && !BF16) {
      if (tiled && ring_fits(cols, num_int, num_fp, ndirty) && ngather <= kRingThreads)
        return launch_tile8_ring(x, rows, cols, cm, l, num_int, num_fp, static_cast<int>(ndirty),
                                 static_cast<int>(ngather), dst, meta, st);
    }
    // bf16 rows beyond 16384 columns (and fp16 ones the ring kernel does not take: more than 512 outlier columns):
    // 180 registers per lane leave room for two workgroups per CU, so the launch is persistent and prefetches the
    // next row (measured at 2048 x 28672: 67 -> 61 us inside the forward; at 2048 x 11008, where three workgroups
    // fit, it is slower)
    if constexpr (BITS == 8) {
      if (tiled && groups > 2048)
        return launch_stream<IdxT, BITS, BF16, 16, kThreads, false, true>(x, rows, cols, cm, l, num_int, num_fp, dst, meta,
                                                                          fp_x, st, tiled);
    }
    if (groups <= 512) QUIK_STREAM(2);
    if (groups <= 1024) QUIK_STREAM(4);
    if (groups <= 2048) QUIK_STREAM(8);
    QUIK_STREAM(16);
#undef QUIK_STREAM
  }
  if (tiled) return QUIK_ERR_SHAPE;  // tile-ordered output exists on the streaming path only
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


// 6-bit operand output through quantize_fp6_wave_kernel; meta: (scale, zero) pairs, or one scale per row (SYM)
template <bool BF16, bool SYM>
int launch_fp6_wave(const void *x, int64_t rows, int64_t cols, const uint8_t *cm, const ColmapLayout &l, int64_t num_int,
                    int64_t num_fp, void *dst, void *meta, hipStream_t st, float sym_divisor = 1.0f) {
  uint32_t words[4];
  if (int rc = colmap_words(cm, cols, num_int, num_fp, st, words)) return rc;
  if ((words[0] & (kColmapStreams | kColmapInPlace)) != (kColmapStreams | kColmapInPlace)) return QUIK_ERR_COLMAP;
  const int nholes = static_cast<int>(words[2]);
  const int J = static_cast<int>((cols / 32 + 63) / 64);
  // one workgroup per CU: as many waves as their row images fit (160 KB of LDS), at most 8 (two per SIMD)
  const int per_cu = 156 / (J * 4) < 8 ? 156 / (J * 4) : 8;
  auto go = [&](auto kern, int W) {
    const int lds = W * J * 4096;  // one row image per wave
    if (lds > 48 * 1024) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
      if (e != hipSuccess) {
        set_last_hip_error(e);
        return static_cast<int>(QUIK_ERR_LAUNCH);
      }
    }
    const int64_t per_xcd = (rows + 7) / 8, groups = (per_xcd + W - 1) / W * 8;
    const int64_t resident = int64_t(num_cus()) * (per_cu / W) / 8 * 8;
    const int grid = static_cast<int>(groups < resident ? groups : resident);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * W), static_cast<size_t>(lds), st, static_cast<const uint16_t *>(x), rows,
                       static_cast<int>(cols), reinterpret_cast<const uint32_t *>(cm + l.off_patch),
                       reinterpret_cast<const uint16_t *>(cm + l.off_fp), nholes,
                       static_cast<int>(num_int), static_cast<int>(num_fp), static_cast<uint8_t *>(dst),
                       static_cast<uint16_t *>(meta), sym_divisor);
    return check_launch();
  };
  // Few rows: workgroups of two waves, so that the launch still reaches every CU (512 rows in workgroups of eight
  // are 64 workgroups, a quarter of the CUs, each taking eight rows in turn).  Measured at 8192 columns, period per
  // launch with two / eight waves: 1280 rows 8.7 / 9.1 us, 1536 rows 9.4 / 9.7, 1792 rows 10.5 / 10.4, 2048 rows
  // 11.7 / 11.5: the switch is at six rows per CU.
  if (rows <= int64_t(6) * num_cus()) {
    switch (J) {
      case 1: return go(quantize_fp6_wave_kernel<BF16, SYM, 1, 2>, 2);
      case 2: return go(quantize_fp6_wave_kernel<BF16, SYM, 2, 2>, 2);
      case 3: return go(quantize_fp6_wave_kernel<BF16, SYM, 3, 2>, 2);
      case 4: return go(quantize_fp6_wave_kernel<BF16, SYM, 4, 2>, 2);
      case 5: return go(quantize_fp6_wave_kernel<BF16, SYM, 5, 2>, 2);
      default: break;
    }
  }
  switch (J) {  // fragments per lane known at compile time: the loops over them unroll
    case 1: return go(quantize_fp6_wave_kernel<BF16, SYM, 1, 8>, 8);
    case 2: return go(quantize_fp6_wave_kernel<BF16, SYM, 2, 8>, 8);
    case 3: return go(quantize_fp6_wave_kernel<BF16, SYM, 3, 8>, 8);
    case 4: return go(quantize_fp6_wave_kernel<BF16, SYM, 4, 8>, 8);
    case 5: return go(quantize_fp6_wave_kernel<BF16, SYM, 5, 7>, 7);
    default: break;
  }
  // longer rows: as many waves as fit one CU's LDS, at least one (rows up to 32768 columns: 64 KB per image)
  if (per_cu >= 4) return go(quantize_fp6_wave_kernel<BF16, SYM, 0, 4>, 4);
  if (per_cu >= 2) return go(quantize_fp6_wave_kernel<BF16, SYM, 0, 2>, 2);
  return go(quantize_fp6_wave_kernel<BF16, SYM, 0, 1>, 1);
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
  colmap_forget(colmap);  // whatever was known about a map at this address is void
  const ColmapLayout l = colmap_layout(cols, num_int, num_fp);
  uint8_t *cm = static_cast<uint8_t *>(colmap);
  uint32_t *mask = reinterpret_cast<uint32_t *>(cm + l.off_mask);
  if (l.idx16) {
    hipLaunchKernelGGL(colmap_build_kernel<uint16_t>, dim3(1), dim3(1024), 0, as_stream(stream), int_indices,
                       num_int, fp_indices, num_fp, cols, reinterpret_cast<uint16_t *>(cm),
                       reinterpret_cast<uint16_t *>(cm + l.off_fp), mask, reinterpret_cast<uint32_t *>(cm + l.off_grp),
                       reinterpret_cast<uint32_t *>(cm + l.off_dirty), reinterpret_cast<uint16_t *>(cm + l.off_slot),
                       reinterpret_cast<uint16_t *>(cm + l.off_kperm), reinterpret_cast<uint32_t *>(cm + l.off_patch),
                       reinterpret_cast<uint16_t *>(cm + l.off_unit), reinterpret_cast<uint16_t *>(cm + l.off_gunit),
                       reinterpret_cast<uint16_t *>(cm + l.off_gcols), reinterpret_cast<uint32_t *>(cm + l.off_flags));
  } else {
    hipLaunchKernelGGL(colmap_build_kernel<uint32_t>, dim3(1), dim3(1024), 0, as_stream(stream), int_indices,
                       num_int, fp_indices, num_fp, cols, reinterpret_cast<uint32_t *>(cm),
                       reinterpret_cast<uint32_t *>(cm + l.off_fp), mask, reinterpret_cast<uint32_t *>(cm + l.off_grp),
                       reinterpret_cast<uint32_t *>(cm + l.off_dirty), reinterpret_cast<uint16_t *>(cm + l.off_slot),
                       reinterpret_cast<uint16_t *>(cm + l.off_kperm), reinterpret_cast<uint32_t *>(cm + l.off_patch),
                       reinterpret_cast<uint16_t *>(cm + l.off_unit), reinterpret_cast<uint16_t *>(cm + l.off_gunit),
                       reinterpret_cast<uint16_t *>(cm + l.off_gcols), reinterpret_cast<uint32_t *>(cm + l.off_flags));
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

extern "C" int quik_colmap_streaming(const void *colmap, int64_t cols, int64_t num_int, int64_t num_fp, void *stream) {
  if (!colmap || cols <= 0 || num_int < 0 || num_fp < 0 || num_int + num_fp != cols) return QUIK_ERR_SHAPE;
  uint32_t flags = 0;
  if (int rc = colmap_flags(colmap, cols, num_int, num_fp, as_stream(stream), &flags)) return rc;
  return (flags & kColmapStreams) ? 1 : 0;
}

extern "C" int quik_asym_quantize_fp6(const void *x, int dtype, int64_t rows, int64_t cols, const void *colmap,
                                      int64_t num_int, int64_t num_fp, void *out6, void *meta, void *stream) {
  if (dtype != QUIK_F16 && dtype != QUIK_BF16) return QUIK_ERR_DTYPE;
  if (rows < 0 || cols <= 0 || num_int <= 0 || num_fp < 0 || num_int + num_fp != cols) return QUIK_ERR_SHAPE;
  if (num_int % 128 != 0 || num_fp % 32 != 0 || cols > kStreamMaxCols) return QUIK_ERR_ALIGN;
  if (rows == 0) return QUIK_OK;
  if (!x || !colmap || !out6 || !meta) return QUIK_ERR_NULL;
  if (reinterpret_cast<uintptr_t>(x) % 16 != 0 || reinterpret_cast<uintptr_t>(out6) % 256 != 0) return QUIK_ERR_ALIGN;
  if (int rc = colmap_require(colmap, cols, num_int, num_fp, as_stream(stream), kColmapStreams | kColmapInPlace)) return rc;
  const ColmapLayout l = colmap_layout(cols, num_int, num_fp);
  const uint8_t *cm = static_cast<const uint8_t *>(colmap);
  hipStream_t st = as_stream(stream);
  return dtype == QUIK_F16 ? launch_fp6_wave<false, false>(x, rows, cols, cm, l, num_int, num_fp, out6, meta, st)
                           : launch_fp6_wave<true, false>(x, rows, cols, cm, l, num_int, num_fp, out6, meta, st);
}

extern "C" int quik_asym_quantize_tile8(const void *x, int dtype, int64_t rows, int64_t cols, const void *colmap,
                                        int64_t num_int, int64_t num_fp, void *out8, void *meta, void *stream) {
  if (dtype != QUIK_F16 && dtype != QUIK_BF16) return QUIK_ERR_DTYPE;
  if (rows < 0 || cols <= 0 || num_int <= 0 || num_fp < 0 || num_int + num_fp != cols) return QUIK_ERR_SHAPE;
  if (num_int % 64 != 0 || num_fp % 32 != 0 || cols > kStreamMaxCols) return QUIK_ERR_ALIGN;
  if (rows == 0) return QUIK_OK;
  if (!x || !colmap || !out8 || !meta) return QUIK_ERR_NULL;
  if (reinterpret_cast<uintptr_t>(x) % 16 != 0 || reinterpret_cast<uintptr_t>(out8) % 256 != 0) return QUIK_ERR_ALIGN;
  uint32_t words[4];
  if (int rc = colmap_words(colmap, cols, num_int, num_fp, as_stream(stream), words)) return rc;
  if (!(words[0] & kColmapStreams)) return QUIK_ERR_COLMAP;
  const ColmapLayout l = colmap_layout(cols, num_int, num_fp);
  const uint8_t *cm = static_cast<const uint8_t *>(colmap);
  hipStream_t st = as_stream(stream);
  return dtype == QUIK_F16 ? launch_asym<uint16_t, 8, false>(x, rows, cols, cm, l, num_int, num_fp, out8, meta, nullptr,
                                                            st, true, words[1], words[3])
                           : launch_asym<uint16_t, 8, true>(x, rows, cols, cm, l, num_int, num_fp, out8, meta, nullptr,
                                                           st, true, words[1], words[3]);
}

extern "C" int quik_sym_quantize_mapped(const void *x, int64_t rows, int64_t cols, const void *colmap, int64_t num_int,
                                        int64_t num_fp, int bits, float divisor, int tiled, void *dst, void *scale,
                                        void *fp_x, void *stream) {
  if (bits != 4 && bits != 8) return QUIK_ERR_BITS;
  if (rows < 0 || cols <= 0 || num_int <= 0 || num_fp < 0 || num_int + num_fp != cols) return QUIK_ERR_SHAPE;
  if (cols % 8 != 0 || cols > kStreamMaxCols || !(divisor > 0.0f)) return QUIK_ERR_SHAPE;
  if (tiled && (num_int % (bits == 4 ? 128 : 64) != 0 || num_fp % 32 != 0)) return QUIK_ERR_ALIGN;
  if (bits == 4 && num_int % 2 != 0) return QUIK_ERR_ALIGN;
  if (rows == 0) return QUIK_OK;
  if (!x || !colmap || !dst || !scale || (!tiled && num_fp > 0 && !fp_x)) return QUIK_ERR_NULL;
  if (reinterpret_cast<uintptr_t>(x) % 16 != 0 || reinterpret_cast<uintptr_t>(dst) % (tiled ? 256 : 1) != 0)
    return QUIK_ERR_ALIGN;
  if (int rc = colmap_require(colmap, cols, num_int, num_fp, as_stream(stream),
                              kColmapStreams | (bits == 4 && tiled ? kColmapInPlace : 0u)))
    return rc;
  const ColmapLayout l = colmap_layout(cols, num_int, num_fp);
  const uint8_t *cm = static_cast<const uint8_t *>(colmap);
  hipStream_t st = as_stream(stream);
  if (bits == 4 && tiled) return launch_fp6_wave<false, true>(x, rows, cols, cm, l, num_int, num_fp, dst, scale, st, divisor);
  return bits == 4 ? launch_sym_stream<4>(x, rows, cols, cm, l, num_int, num_fp, dst, scale, fp_x, st, tiled != 0, divisor)
                   : launch_sym_stream<8>(x, rows, cols, cm, l, num_int, num_fp, dst, scale, fp_x, st, tiled != 0, divisor);
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
