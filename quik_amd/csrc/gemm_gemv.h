// MixedQLinear forward for very few token rows (single-stream decode; the host uses it for one and two): a
// matrix-vector product per token row, bound by one pass over the weights.
//
// With so few token rows a 32-row MFMA block is mostly padding, and what the weight-streaming MFMA kernel
// (gemm_decode.h) does around the MFMAs (LDS transpose of every weight chunk, partial sums of eight waves meeting
// in LDS at every slab end, four barriers per slab) costs more than the products.  Here a WAVE owns whole output
// columns: it streams a column's weight row with 16-byte loads (1 KB per instruction, whole lines), multiplies with
// the packed dot-product instructions (v_dot8_i32_i4 / v_dot4_i32_i8: the codes of both operands are two's
// complement nibbles / bytes in the same element order) against the token rows' codes, which every workgroup
// keeps in LDS (at most 4 x K bytes, copied once), and sums over the wave at the column's end.  No barrier after the
// copy of the token rows, no cross-wave sums.  The outlier columns (fp16 / bf16 weights and values) travel through
// the same stream of loads as further 16-byte pieces of the column, kGemvPieces pieces ahead, across column
// boundaries; a column's three epilogue scalars wait in a small LDS table that the workgroup fills at the start.
// Integer sums are exact; the fp32 outlier sum is taken in lane order, then over the wave.  Epilogue as in the other
// fused kernels: (f32(acc) (s_row s_col) + outliers) + (zs w_red + bias).
//
// QUANT: the kernel also quantises the token rows itself (one launch per forward).  Every workgroup does it for all
// of the (at most kGemvMaxRows) rows, redundantly: a row is a few KB out of L2, against a launch and a trip through
// memory for the codes that the two-launch form pays.  Same arithmetic as the quantize kernels (quantize_math.h):
// min / max over the integer columns, scale, zero, the codes of every group of 8 source columns written to a staging
// area in source order, then squeezed into the compact order of the weights' K axis through the column map's unit
// tables (colmap.h); outlier values in the caller's order.  Codes and scales are bit-identical to the quantize
// kernels', so the output is bit-identical to the two-launch form.  Symmetric activations (fp16): the largest |x|
// in place of min / max, scale = fp16(max |x| / divisor), codes rne(fp16(x / scale)), no zero-point term
// (reference: experiments/qlinear.py:97-103, src/symmetric/symmetric.cu:6-61).
#pragma once
#include "gemm_kernels.h"
#include "quantize_math.h"

namespace quik {

constexpr int kGemvWaves = 8;
// 16-byte loads in flight per lane.  Measured (forward with cold weights, 13B / 70B gate_proj at one row): 2: 14.2 /
// 29.5 us, 3: 13.2 / 28.3, 4: 12.7 / 28.0, 6: 13.2 / 28.6, 8: 14.0 / 28.8, 12: 15.6 / 27.9, 16: 16.8 / 30.3
constexpr int kGemvPieces = 4;

// LDS: the token rows' codes, MT rows of `xstride` bytes (whole kilobytes), then their outlier values, MT rows of
// `fstride` bytes
__host__ __device__ inline int64_t gemv_xstride(int64_t kbytes) { return (kbytes + 1023) / 1024 * 1024; }
__host__ __device__ inline int64_t gemv_fstride(int64_t F) { return (F * 2 + 1023) / 1024 * 1024; }
__host__ __device__ inline int64_t gemv_smem(int mt, int64_t kbytes, int64_t F) { return mt * (gemv_xstride(kbytes) + gemv_fstride(F)); }
// behind them: the epilogue scalars (column scale, reduced weight, bias, one spare) of the workgroup's own columns,
// 8 bytes per column, `iters` rounds of kGemvWaves columns
__host__ __device__ inline int64_t gemv_table_bytes(int64_t iters) { return iters * kGemvWaves * 8; }

// what the QUANT form needs beside FusedArgs (whose qx, meta and fp_x it does not read): the activations and the
// column map's tables
struct GemvQuant {
  const uint16_t *x, *fp_col, *unit, *gather_unit, *gather_cols;
  const uint32_t *grp;
  int cols, num_int, num_fp, ngather;
  float sym_divisor;  // symmetric activations only: scale = fp16(max |x| / sym_divisor)
};
// LDS of the QUANT form behind the token rows' codes and the scalars' table: the raw row (2 bytes per column), the
// column map's group words (4 bytes per 8 columns) and unit words (2 bytes per 16 integer columns), each in whole
// kilobytes (they arrive as 1 KB direct copies), the staging area (one code byte per source column + 32 spare) and
// the reduction slots
struct GemvQuantLds {
  int64_t raw, grp, unit, stage, red, bytes;  // offsets from the area's start, total
};
__host__ __device__ inline GemvQuantLds gemv_quant_lds(int64_t cols, int64_t num_int) {
  auto kb = [](int64_t v) { return (v + 1023) / 1024 * 1024; };
  GemvQuantLds l;
  l.raw = 0;
  l.grp = l.raw + kb(cols * 2);
  l.unit = l.grp + kb(cols / 8 * 4);
  l.stage = l.unit + kb(num_int / 16 * 2);
  l.red = l.stage + (cols + 47) / 16 * 16;
  l.bytes = l.red + 4 * kGemvWaves * 4;
  return l;
}

// 1 KB direct copies global -> LDS of `bytes` bytes (a multiple of 16, at least 16) by the workgroup's waves; lanes
// past the end repeat the last 16 bytes
__device__ __forceinline__ void gemv_copy_in(const void *src, int bytes, uint32_t lds_addr, int wave, int lane) {
  for (int q = wave; q < (bytes + 1023) >> 10; q += kGemvWaves) {
    int off = (q << 10) + lane * 16;
    off = off < bytes ? off : bytes - 16;
    dma_load16(static_cast<const uint8_t *>(src), static_cast<uint32_t>(off), lds_addr + (q << 10));
  }
}

// One token row (already in LDS as `raw`) -> codes in compact order (xs_row: K bytes, or K / 2 for 4 bits) and outlier
// values (fs_row), by all threads of the workgroup; returns the row's scale and zero as the kernels read them from
// `meta`.  grp_s / unit_s: the column map's tables in LDS; goff / gunit / fcol: this thread's gathered unit (its 16
// source columns, two per register) and outlier column.
template <int BITS, bool BF16, bool SYM>
__device__ __forceinline__ void gemv_quantize_row(const uint8_t *raw, const uint32_t *grp_s, const uint16_t *unit_s,
                                                  const GemvQuant &q, const uint32_t (&goff)[8], int gunit, int fcol,
                                                  uint8_t *xs_row, uint8_t *fs_row, uint8_t *stage, float *red,
                                                  float &scale_out, float &zero_out) {
  constexpr int T = kGemvWaves * 64;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int nvec = q.cols >> 3;
  const float inf = __builtin_inff();
  // min / max over the integer columns (a group's low word byte marks its outlier columns)
  float mn = inf, mx = -inf;
  for (int g = tid; g < nvec; g += T) {
    const uint4 v = *reinterpret_cast<const uint4 *>(raw + g * 16);
    const uint32_t skip = grp_s[g] & 0xFFu;
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint16_t hbits = static_cast<uint16_t>(w[e >> 1] >> (16 * (e & 1)));
      const bool out = (skip >> e) & 1u;
      if constexpr (SYM) {
        // largest |x| as a bit pattern (non-negative fp16 patterns order like integers, NaN patterns above infinity);
        // a 15-bit integer is exact as a float, so the float reductions below carry it
        mx = fmaxf(mx, out ? 0.0f : static_cast<float>(hbits & 0x7FFFu));
      } else {
        const float f = to_f32<BF16>(hbits);
        mn = fminf(mn, out ? inf : f);
        mx = fmaxf(mx, out ? -inf : f);
      }
    }
  }
  mn = wave_min(mn);
  mx = wave_max(mx);
  if (lane == 0) {
    red[wave] = mn;
    red[kGemvWaves + wave] = mx;
  }
  __syncthreads();
  mn = red[0];
  mx = red[kGemvWaves];
#pragma unroll
  for (int w = 1; w < kGemvWaves; ++w) {
    mn = fminf(mn, red[w]);
    mx = fmaxf(mx, red[kGemvWaves + w]);
  }
  RowQuant<BF16> rq;
  if constexpr (SYM) {
    rq.init_sym(static_cast<uint32_t>(mx), q.sym_divisor);
  } else {
    rq.init(mn, mx, BITS);
  }
  scale_out = to_f32<BF16>(rq.scale_bits);
  zero_out = to_f32<BF16>(rq.zero_bits);
  // codes of every group, source order; outlier values in the caller's order
  const bool slow = __builtin_amdgcn_readfirstlane(rq.slow ? 1 : 0);
  for (int g = tid; g < nvec; g += T) {
    const uint4 v = *reinterpret_cast<const uint4 *>(raw + g * 16);
    const uint2 c = slow ? group_codes<BITS, BF16, true, SYM>(v, rq) : group_codes<BITS, BF16, false, SYM>(v, rq);
    *reinterpret_cast<uint2 *>(stage + g * 8) = c;
  }
  if (tid < q.num_fp) reinterpret_cast<uint16_t *>(fs_row)[tid] = reinterpret_cast<const uint16_t *>(raw)[fcol];
  __syncthreads();
  // 16-column units of the compact order: 16 consecutive staged bytes from the unit's first column on, or a gather
  auto put = [&](int u, const uint4 &c) __attribute__((always_inline)) {
    if constexpr (BITS == 8) {
      *reinterpret_cast<uint4 *>(xs_row + u * 16) = c;
    } else {
      // byte pairs (c0, c1) -> c0 | c1 << 4: t = w | w >> 4 leaves them in bytes 0 and 2
      const uint32_t t0 = c.x | (c.x >> 4), t1 = c.y | (c.y >> 4), t2 = c.z | (c.z >> 4), t3 = c.w | (c.w >> 4);
      *reinterpret_cast<uint2 *>(xs_row + u * 8) =
          make_uint2(__builtin_amdgcn_perm(t1, t0, 0x06040200u), __builtin_amdgcn_perm(t3, t2, 0x06040200u));
    }
  };
  const int nu = q.num_int >> 4;
  for (int u = tid; u < nu; u += T) {
    const uint32_t c0 = unit_s[u];
    if (c0 != 0xFFFFu) {
      // two aligned 16-byte reads, a shift by whole words (bit-mask selects) and by bytes
      const uint4 a = *reinterpret_cast<const uint4 *>(stage + (c0 & ~15u));
      const uint4 b = *reinterpret_cast<const uint4 *>(stage + (c0 & ~15u) + 16);
      uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
      const uint32_t by2 = 0u - ((c0 >> 3) & 1u), by1 = 0u - ((c0 >> 2) & 1u);
#pragma unroll
      for (int t = 0; t < 6; ++t) w[t] = (w[t + 2] & by2) | (w[t] & ~by2);
#pragma unroll
      for (int t = 0; t < 5; ++t) w[t] = (w[t + 1] & by1) | (w[t] & ~by1);
      put(u, make_uint4(__builtin_amdgcn_alignbyte(w[1], w[0], c0), __builtin_amdgcn_alignbyte(w[2], w[1], c0),
                        __builtin_amdgcn_alignbyte(w[3], w[2], c0), __builtin_amdgcn_alignbyte(w[4], w[3], c0)));
    }
  }
  if (tid < q.ngather) {
    uint32_t c[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const uint32_t b0 = stage[goff[2 * t] & 0xFFFFu], b1 = stage[goff[2 * t] >> 16];
      const uint32_t b2 = stage[goff[2 * t + 1] & 0xFFFFu], b3 = stage[goff[2 * t + 1] >> 16];
      c[t] = b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
    }
    put(gunit, make_uint4(c[0], c[1], c[2], c[3]));
  }
  __syncthreads();  // (the raw row, the staging area and the reduction slots are free for the next row)
}

// Sums over the wave in a fixed order (every lane active), result in every lane: four DPP steps make each row of 16
// uniform, two row broadcasts (lane 15 of a row into the next row, lane 31 into the upper half) leave the total in
// the last row, one scalar read hands it out.  (Four scalar reads and three scalar adds instead of the broadcasts
// cost more here: every read of a vector register that a DPP instruction has just written waits out a hazard.)
constexpr int kDppRowBcast15 = 0x142, kDppRowBcast31 = 0x143;
__device__ __forceinline__ int32_t wave_total(int32_t v) {
  v += dpp_move_i<kDppSwap1>(v);
  v += dpp_move_i<kDppSwap2>(v);
  v += dpp_move_i<kDppHalfMirror>(v);
  v += dpp_move_i<kDppMirror>(v);
  v += __builtin_amdgcn_update_dpp(0, v, kDppRowBcast15, 0xA, 0xF, false);
  v += __builtin_amdgcn_update_dpp(0, v, kDppRowBcast31, 0xC, 0xF, false);
  return __builtin_amdgcn_readlane(v, 63);
}
__device__ __forceinline__ float wave_total(float v) {
  v += dpp_move<kDppSwap1>(v);
  v += dpp_move<kDppSwap2>(v);
  v += dpp_move<kDppHalfMirror>(v);
  v += dpp_move<kDppMirror>(v);
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kDppRowBcast15, 0xA, 0xF, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kDppRowBcast31, 0xC, 0xF, false));
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// QUANT: kGemvNoQuant (the token rows' codes come from a quantize launch), kGemvAsym / kGemvSym (quantised here)
constexpr int kGemvNoQuant = 0, kGemvAsym = 1, kGemvSym = 2;
template <int MODE, bool BF16, int MT, int QUANT = kGemvNoQuant>
__global__ __launch_bounds__(kGemvWaves * 64) void gemv_decode_kernel(FusedArgs args, GemvQuant quant) {
  static_assert(MODE == kInt4 || MODE == kInt8, "integer codes");
  static_assert(QUANT != kGemvSym || !BF16, "symmetric activations are fp16");
  struct {
    const uint8_t *qx, *qw;
    const uint16_t *meta, *s_col, *w_red, *fp_x, *fp_w, *bias;
    uint16_t *out;
    int M, N, ldo, kbytes, F, meta_stride;
    float shift;
  } p;
  p.qx = args.qx, p.qw = args.qw, p.meta = args.meta, p.s_col = args.s_col, p.w_red = args.w_red;
  p.fp_x = args.fp_x, p.fp_w = args.fp_w, p.bias = args.bias, p.out = args.out;
  p.M = args.M, p.N = args.N, p.ldo = args.ldo, p.kbytes = args.kbytes, p.F = args.F;
  p.meta_stride = args.meta_stride, p.shift = args.shift;
  extern __shared__ __align__(16) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kbytes = p.kbytes, fbytes = p.F * 2;
  const int xstride = static_cast<int>(gemv_xstride(kbytes)), fstride = static_cast<int>(gemv_fstride(p.F));
  const int ipieces = xstride >> 10, fpieces = fstride >> 10;  // 1 KB pieces of a column: codes, outlier weights
  const int pieces = ipieces + fpieces;
  uint8_t *xs = smem, *fs = smem + MT * xstride;

  // ---- the stream's first loads go out before anything that waits: they do not depend on the token rows
  const int step = gridDim.x * kGemvWaves;
  const int n_first = blockIdx.x * kGemvWaves + wave;
  const uint8_t *fw = fbytes > 0 ? reinterpret_cast<const uint8_t *>(p.fp_w) : p.qw;
  const int frow = fbytes > 0 ? fbytes : kbytes;
  int ld_n = n_first, ld_p = 0;  // next item to load
  // Every item is ONE unconditional 16-byte load from a wave-uniform base plus a lane offset (with loads under a
  // branch the number in flight is unknown at compile time and every wait becomes a wait for all of them).
  auto issue = [&](v4i &b) __attribute__((always_inline)) {
    const int n = ld_n < p.N ? ld_n : p.N - 1;  // past the last column: any valid one, never stored
    const bool is_int = ld_p < ipieces;
    const uint8_t *base = is_int ? p.qw + int64_t(n) * kbytes : fw + int64_t(n) * frow;      // wave-uniform
    const int q = is_int ? ld_p : ld_p - ipieces, row_bytes = is_int ? kbytes : frow;
    int off = (q << 10) + lane * 16;
    off = off < row_bytes ? off : row_bytes - 16;  // past the row's end: a repeated piece, masked where it is used
    b = *reinterpret_cast<const v4i *>(base + off);
    if (++ld_p == pieces) {
      ld_p = 0;
      ld_n += step;
    }
  };
  v4i buf[kGemvPieces];
  auto first_pieces = [&]() __attribute__((always_inline)) {
    static_for<kGemvPieces - 1>([&](auto I) __attribute__((always_inline)) { issue(buf[I.value]); });
  };

  float srow = 0.0f, zs = 0.0f;  // lane m keeps token row m's scale and zero-point term
  if constexpr (QUANT != kGemvNoQuant) {
    // ---- token rows -> codes and outlier values in LDS, quantised here.  The first row and the column map's
    // tables arrive together as direct copies; this thread's gathered unit and outlier column go to registers
    // (unconditional loads from clamped indices: under conditions each would wait for the one before it).
    // These few kilobytes are requested IN FRONT of the first weight pieces: a wave's loads are counted in the
    // order of issue, and behind the pieces (32 KB per workgroup, every workgroup of the launch at once) the row
    // would count as landed only after that whole burst, with the quantize work still to come.
    uint8_t *area = smem + MT * (xstride + fstride) + gemv_table_bytes((p.N + step - 1) / step);
    const GemvQuantLds ql = gemv_quant_lds(quant.cols, quant.num_int);
    const uint32_t area_lds = lds_address(area);
    gemv_copy_in(quant.x, quant.cols * 2, area_lds + ql.raw, wave, lane);
    gemv_copy_in(quant.grp, (quant.cols >> 3) * 4, area_lds + ql.grp, wave, lane);
    gemv_copy_in(quant.unit, (quant.num_int >> 4) * 2, area_lds + ql.unit, wave, lane);
    const uint16_t *spare = reinterpret_cast<const uint16_t *>(quant.grp);  // (always there; the other tables may be empty)
    const bool has_g = tid < quant.ngather, has_f = tid < quant.num_fp;
    const int gunit = *(has_g ? quant.gather_unit + tid : spare);
    const uint4 ga = reinterpret_cast<const uint4 *>(has_g ? quant.gather_cols + 16 * tid : spare)[0];
    const uint4 gb = reinterpret_cast<const uint4 *>(has_g ? quant.gather_cols + 16 * tid : spare)[1];
    const uint32_t goff[8] = {ga.x, ga.y, ga.z, ga.w, gb.x, gb.y, gb.z, gb.w};
    const int fcol = *(has_f ? quant.fp_col + tid : spare);
    __builtin_amdgcn_sched_barrier(0);
    first_pieces();
    __builtin_amdgcn_sched_barrier(0);
    for (int m = 0; m < p.M; ++m) {
      // A second row takes the first one's place (both requested at once at the start were no faster, measured, and
      // cost a second row of LDS); it sits behind the weight pieces, which have long landed by then.
      if (m > 0) gemv_copy_in(quant.x + int64_t(m) * quant.cols, quant.cols * 2, area_lds + ql.raw, wave, lane);
      // the first row: everything but the weight pieces, which were issued last
      if (m == 0) __builtin_amdgcn_s_waitcnt(vmcnt_imm(kGemvPieces - 1));
      else __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
      __syncthreads();
      float sc, zr;
      gemv_quantize_row<MODE == kInt4 ? 4 : 8, BF16, QUANT == kGemvSym>(area + ql.raw, reinterpret_cast<const uint32_t *>(area + ql.grp),
                                                     reinterpret_cast<const uint16_t *>(area + ql.unit), quant, goff,
                                                     gunit, fcol, xs + m * xstride, fs + m * fstride, area + ql.stage,
                                                     reinterpret_cast<float *>(area + ql.red), sc, zr);
      if (lane == m) {
        srow = sc;
        zs = QUANT == kGemvSym ? 0.0f : zr + p.shift * sc;  // (symmetric: no zero-point term)
      }
    }
  } else {
    first_pieces();
    // ---- token rows -> LDS (codes, outlier values) with direct copies, 1 KB each.  Rows past M repeat the last one
    // (their results are never stored); lanes past a row's end repeat its last 16 bytes (the weight pieces that
    // stand against them are masked to zero where they are used).
    const uint32_t lds0 = lds_address(smem);
    for (int u = wave; u < MT * ipieces; u += kGemvWaves) {  // (wave-uniform)
      const int m = u / ipieces, q = u - m * ipieces, mm = m < p.M ? m : p.M - 1;
      int off = (q << 10) + lane * 16;
      off = off < kbytes ? off : kbytes - 16;
      dma_load16(p.qx, static_cast<uint32_t>(mm * kbytes + off), lds0 + m * xstride + (q << 10));
    }
    for (int u = wave; u < MT * fpieces; u += kGemvWaves) {
      const int m = u / fpieces, q = u - m * fpieces, mm = m < p.M ? m : p.M - 1;
      int off = (q << 10) + lane * 16;
      off = off < fbytes ? off : fbytes - 16;
      dma_load16(reinterpret_cast<const uint8_t *>(p.fp_x), static_cast<uint32_t>(mm * fbytes + off),
                 lds0 + MT * xstride + m * fstride + (q << 10));
    }
    const int m = lane < p.M ? lane : p.M - 1;
    srow = to_f32<BF16>(p.meta[int64_t(m) * p.meta_stride]);
    zs = p.w_red ? to_f32<BF16>(p.meta[2 * int64_t(m) + 1]) + p.shift * srow : 0.0f;
  }

  // ---- the epilogue scalars of the workgroup's columns -> LDS (a few hundred bytes; read back at each column's end,
  // so that no global load whose result is needed at once sits between the pieces in flight)
  uint16_t *table = reinterpret_cast<uint16_t *>(smem + MT * (xstride + fstride));
  {
    const int step_ = step;
    const int iters = (p.N - blockIdx.x * kGemvWaves + step_ - 1) / step_;
    for (int j = tid; j < iters * kGemvWaves * 3; j += kGemvWaves * 64) {
      const int col = j / 3, k = j - col * 3;
      const int nn = blockIdx.x * kGemvWaves + (col & (kGemvWaves - 1)) + (col / kGemvWaves) * step_;
      // (one unconditional load: under conditions each array's load would wait for the one before it)
      const uint16_t *src = k == 0 ? p.s_col : k == 1 ? (p.w_red ? p.w_red : p.s_col) : (p.bias ? p.bias : p.s_col);
      const uint16_t v = src[nn < p.N ? nn : p.N - 1];
      table[col * 4 + k] = (k == 1 && !p.w_red) || (k == 2 && !p.bias) ? uint16_t(0) : v;
    }
  }

  // ---- the stream: this wave's columns n_first, n_first + step, ..., `pieces` items each
  int n = n_first, piece = 0;  // the item being consumed
  int32_t acc[MT];
  float accf[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) acc[m] = 0, accf[m] = 0.0f;
  int it = 0;  // how many columns this wave has finished
  auto consume = [&](const v4i &b_) __attribute__((always_inline)) {
    if (piece < ipieces) {
      const uint8_t *xp = xs + (piece << 10) + lane * 16;
      const int keep = (piece << 10) + lane * 16 < kbytes ? -1 : 0;  // past the row's end: a repeated piece
      const v4i b = v4i{b_.x & keep, b_.y & keep, b_.z & keep, b_.w & keep};
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        const v4i x = *reinterpret_cast<const v4i *>(xp + m * xstride);
        if constexpr (MODE == kInt4) {
          acc[m] = __builtin_amdgcn_sdot8(x.x, b.x, acc[m], false);
          acc[m] = __builtin_amdgcn_sdot8(x.y, b.y, acc[m], false);
          acc[m] = __builtin_amdgcn_sdot8(x.z, b.z, acc[m], false);
          acc[m] = __builtin_amdgcn_sdot8(x.w, b.w, acc[m], false);
        } else {
          acc[m] = __builtin_amdgcn_sdot4(x.x, b.x, acc[m], false);
          acc[m] = __builtin_amdgcn_sdot4(x.y, b.y, acc[m], false);
          acc[m] = __builtin_amdgcn_sdot4(x.z, b.z, acc[m], false);
          acc[m] = __builtin_amdgcn_sdot4(x.w, b.w, acc[m], false);
        }
      }
    } else {
      const int off = ((piece - ipieces) << 10) + lane * 16;
      const bool live = off < fbytes;  // (lanes past the outlier columns hold a repeated piece)
      const uint32_t w[4] = {static_cast<uint32_t>(b_.x), static_cast<uint32_t>(b_.y), static_cast<uint32_t>(b_.z),
                             static_cast<uint32_t>(b_.w)};
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        const v4i xv = *reinterpret_cast<const v4i *>(fs + m * fstride + (live ? off : 0));
        const uint32_t x[4] = {static_cast<uint32_t>(xv.x), static_cast<uint32_t>(xv.y), static_cast<uint32_t>(xv.z),
                               static_cast<uint32_t>(xv.w)};
        float t = 0.0f;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          // fp32 products of 16-bit values are exact; one rounding per addition
          t = __builtin_fmaf(to_f32<BF16>(static_cast<uint16_t>(x[k])), to_f32<BF16>(static_cast<uint16_t>(w[k])), t);
          t = __builtin_fmaf(to_f32<BF16>(static_cast<uint16_t>(x[k] >> 16)), to_f32<BF16>(static_cast<uint16_t>(w[k] >> 16)), t);
        }
        accf[m] += live ? t : 0.0f;
      }
    }
    if (++piece == pieces) {
      // the column is complete: sums over the wave, epilogue by lanes 0 .. M-1 (one token row each)
      const uint2 e = *reinterpret_cast<const uint2 *>(table + (it * kGemvWaves + wave) * 4);
      const float sc = to_f32<BF16>(static_cast<uint16_t>(e.x));
      const float wr = to_f32<BF16>(static_cast<uint16_t>(e.x >> 16)), bs = to_f32<BF16>(static_cast<uint16_t>(e.y));
      int32_t ti = 0;
      float tf = 0.0f;
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        const int32_t si = wave_total(acc[m]);
        const float sf = wave_total(accf[m]);
        ti = lane == m ? si : ti;
        tf = lane == m ? sf : tf;
        acc[m] = 0;
        accf[m] = 0.0f;
      }
      if (lane < p.M) {
        const float val = (static_cast<float>(ti) * (srow * sc) + tf) + (zs * wr + bs);
        p.out[int64_t(lane) * p.ldo + n] = from_f32<BF16>(val);
      }
      piece = 0;
      n += step;
      ++it;
    }
  };

  __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));  // the token rows (and the first pieces) have landed
  __syncthreads();
  while (n < p.N) {  // (a wave's own column sequence; nothing is shared between the waves any more)
    static_for<kGemvPieces>([&](auto I) __attribute__((always_inline)) {
      constexpr int i = I.value;
      issue(buf[(i + kGemvPieces - 1) % kGemvPieces]);
      if (n < p.N) consume(buf[i]);
    });
  }
}

}  // namespace quik
