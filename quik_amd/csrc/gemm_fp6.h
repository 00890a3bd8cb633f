// int4 x int4 GEMM on the 6-bit matrix-core path of CDNA4 (gfx950), exact.
//
// v_mfma_f32_32x32x64_f8f6f4 with 6-bit E2M3 operands runs at twice the rate of the int8 MFMA.
// The E2M3 bit patterns 0 .. 15 (sign 0, exponent 00 / 01) are the uniformly spaced values
// L / 8, so a 4-bit level L = code + 8 IS an E2M3 number, zero-extended to 6 bits.  Products
// La Lw / 64 are multiples of 1/64 and their sum over K stays below 2^15 for K < 131072, so the
// fp32 accumulation is exact, and
//     sum_k a_k w_k = 64 S - 8 sum_k La_k - 8 sum_k Lw_k + 64 K,      S = sum_k (La_k / 8)(Lw_k / 8)
// recovers the integer accumulator exactly (every term is an integer below 2^24).  From there
// the epilogue is the one of gemm_kernels.h, so the output is bit-identical to the int8-MFMA path.
//
// Operand format: fp6_format.h (heads [R][K/128][64 bytes], tails plane-major, level sums).  One MFMA
// k-step (64 elements) of a lane is fragment 2 s + h of a 128-element block: the head is one 16-byte
// LDS read, the tail one 8-byte read, both conflict-free.
//
// Pipeline: a ring of 6 LDS slots, one per k-step, filled by global_load_lds_dwordx4.  While step j
// feeds the MFMAs, the fragments of step j + 1 are read into registers, steps j + 2 .. j + 4 are
// landing and step j + 5 is being issued; the outlier GEMM's fp16/bf16 steps (16 elements each,
// same 32 bytes per row) run through the same ring after the integer steps.
#pragma once
#include "fp6_format.h"
#include "gemm_kernels.h"

namespace quik {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v8i __attribute__((ext_vector_type(8)));

template <class C>
struct Fp6Pipe {
  static constexpr int MI = C::MI, NI = C::NI, NS = 6, NF = MI + NI;
  // per step: heads (BM + BN) x 32 bytes, tails 2 planes x (BM + BN) x 8 bytes
  static constexpr int XH = C::BM * 32, WH = C::BN * 32, XT = C::BM * 16, WT = C::BN * 16;
  static constexpr int XH_OFF = 0, WH_OFF = XH, XT_OFF = XH + WH, WT_OFF = XH + WH + XT;
  static constexpr int STAGE = XH + WH + XT + WT;
  static constexpr int SMEM = NS * STAGE;
  static constexpr int per_wave(int bytes) { return (bytes / 1024 + C::WAVES - 1) / C::WAVES; }
  static constexpr int XH_I = per_wave(XH), WH_I = per_wave(WH), XT_I = per_wave(XT), WT_I = per_wave(WT);
  static constexpr int P = XH_I + WH_I + XT_I + WT_I;  // loads per wave and step
  static_assert(3 * P <= 63, "three steps in flight must fit the vmcnt counter");

  uint8_t *smem;
  uint32_t lds0;
  int wave;
  const uint8_t *Xh, *Wh, *Xt, *Wt;      // set 0: heads / tails of the integer operands
  const uint8_t *Xf, *Wf;                // set 1: fp16 / bf16 outlier operands
  int64_t xt_plane, wt_plane;            // bytes from one tail plane to the next
  uint32_t vxh[XH_I], vwh[WH_I], vxt[XT_I], vwt[WT_I], vxf[XH_I], vwf[WH_I];
  int steps0, steps;                     // steps of set 0, of both sets
  int x_head, w_head, x_tail, w_tail;    // this lane's fragment offsets inside a slot

  // heads / outlier rows: 32 bytes per row and step, two 16-byte chunks; lane -> (row = lane / 2, chunk = lane % 2);
  // chunk c of row r sits in slot c ^ ((r >> 2) & 1): eight consecutive lanes of a 16-byte read then cover all
  // eight 16-byte bank groups
  __device__ __forceinline__ void init(uint8_t *smem_, const uint8_t *xbuf, const Fp6Layout &lx, const uint8_t *wbuf,
                                       const Fp6Layout &lw, int m0, int n0, int rows_x, int rows_w,
                                       const uint8_t *fx, const uint8_t *fw, int fbytes) {
    smem = smem_;
    lds0 = lds_address(smem_);
    const int lane = threadIdx.x & 63;
    wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;
    const int64_t ldx = lx.kblocks * 64, ldw = lw.kblocks * 64;
    Xh = xbuf + int64_t(m0) * ldx;
    Wh = wbuf + int64_t(n0) * ldw;
    Xt = xbuf + lx.tails_off + int64_t(m0) * 8;
    Wt = wbuf + lw.tails_off + int64_t(n0) * 8;
    xt_plane = lx.rows_pad * 8;
    wt_plane = lw.rows_pad * 8;
    Xf = fx, Wf = fw;
    const int lrow = lane >> 1;
    const int gchunk = (lane & 1) ^ ((lrow >> 2) & 1);
    auto head_off = [&](int instr, int total, int rows_valid, int64_t ld) {
      const int i = instr < total ? instr : total - 1;  // surplus waves repeat the last load
      const int row = i * 32 + lrow;
      return static_cast<uint32_t>((row < rows_valid ? row : rows_valid - 1) * ld + gchunk * 16);
    };
#pragma unroll
    for (int j = 0; j < XH_I; ++j) {
      vxh[j] = head_off(wave * XH_I + j, XH / 1024, rows_x, ldx);
      vxf[j] = head_off(wave * XH_I + j, XH / 1024, rows_x, fbytes);
    }
#pragma unroll
    for (int j = 0; j < WH_I; ++j) {
      vwh[j] = head_off(wave * WH_I + j, WH / 1024, rows_w, ldw);
      vwf[j] = head_off(wave * WH_I + j, WH / 1024, rows_w, fbytes);
    }
    // tails: a plane holds 8 bytes per row; one load covers 128 rows; loads [0, BM/128) are plane h = 0
    auto tail_off = [&](int instr, int rows_tile, int64_t plane) {
      const int per_plane = rows_tile / 128 > 0 ? rows_tile / 128 : 1;
      const int total = 2 * per_plane;
      const int i = instr < total ? instr : total - 1;
      const int h = i / per_plane, part = i % per_plane;
      return static_cast<uint32_t>(h * plane + (part * 128) * 8 + lane * 16);
    };
#pragma unroll
    for (int j = 0; j < XT_I; ++j) vxt[j] = tail_off(wave * XT_I + j, C::BM, xt_plane);
#pragma unroll
    for (int j = 0; j < WT_I; ++j) vwt[j] = tail_off(wave * WT_I + j, C::BN, wt_plane);
    steps0 = static_cast<int>(lx.kblocks) * 2;
    steps = steps0 + fbytes / 32;
    const int r = lane & 31, h = lane >> 5;
    x_head = XH_OFF + (wm * C::WM + r) * 32 + ((h ^ ((r >> 2) & 1)) << 4);
    w_head = WH_OFF + (wn * C::WN + r) * 32 + ((h ^ ((r >> 2) & 1)) << 4);
    x_tail = XT_OFF + (h * C::BM + wm * C::WM + r) * 8;
    w_tail = WT_OFF + (h * C::BN + wn * C::WN + r) * 8;
  }

  // LDS destination of load `instr` of an operand region (surplus loads repeat the last one)
  template <int IDX>
  __device__ __forceinline__ void issue_one(int step) const {
    const int st = step < steps ? step : steps - 1;
    const uint32_t slot = lds0 + (step % NS) * STAGE;
    const bool second = st >= steps0;
    const int s0 = second ? steps0 - 1 : st;          // tails of outlier steps: a harmless re-load
    const int64_t hb = second ? int64_t(st - steps0) * 32 : int64_t(st) * 32;
    if constexpr (IDX < XH_I) {
      const int i = wave * XH_I + IDX;
      const int total = XH / 1024;
      dma_load16((second ? Xf : Xh) + hb, second ? vxf[IDX] : vxh[IDX], slot + XH_OFF + (i < total ? i : total - 1) * 1024);
    } else if constexpr (IDX < XH_I + WH_I) {
      constexpr int J = IDX - XH_I;
      const int i = wave * WH_I + J;
      const int total = WH / 1024;
      dma_load16((second ? Wf : Wh) + hb, second ? vwf[J] : vwh[J], slot + WH_OFF + (i < total ? i : total - 1) * 1024);
    } else if constexpr (IDX < XH_I + WH_I + XT_I) {
      constexpr int J = IDX - XH_I - WH_I;
      const int i = wave * XT_I + J;
      const int total = XT / 1024;
      dma_load16(Xt + int64_t(s0) * 2 * xt_plane, vxt[J], slot + XT_OFF + (i < total ? i : total - 1) * 1024);
    } else {
      constexpr int J = IDX - XH_I - WH_I - XT_I;
      const int i = wave * WT_I + J;
      const int total = WT / 1024;
      dma_load16(Wt + int64_t(s0) * 2 * wt_plane, vwt[J], slot + WT_OFF + (i < total ? i : total - 1) * 1024);
    }
  }
  template <int FIRST, int COUNT>
  __device__ __forceinline__ void issue_range(int step) const {
    if constexpr (COUNT > 0) {
      issue_one<FIRST>(step);
      issue_range<FIRST + 1, COUNT - 1>(step);
    }
  }
  __device__ __forceinline__ void issue(int step) const { issue_range<0, P>(step); }

  // Fill the ring: afterwards steps 0 and 1 are visible and steps 2 .. 4 are in flight.
  __device__ __forceinline__ void start() const {
    issue(0);
    issue(1);
    issue(2);
    issue(3);
    issue(4);
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(3 * P));
    __syncthreads();
  }

  __device__ __forceinline__ void read6(int step, v4i (&fh)[NF], v2i (&ft)[NF]) const {
    const uint8_t *s = smem + (step % NS) * STAGE;
#pragma unroll
    for (int j = 0; j < NF; ++j) {
      const int ho = j < MI ? x_head + j * 32 * 32 : w_head + (j - MI) * 32 * 32;
      const int to = j < MI ? x_tail + j * 32 * 8 : w_tail + (j - MI) * 32 * 8;
      fh[j] = *reinterpret_cast<const v4i *>(s + ho);
      ft[j] = *reinterpret_cast<const v2i *>(s + to);
    }
  }
  __device__ __forceinline__ void read16(int step, v4i (&f)[NF]) const {
    const uint8_t *s = smem + (step % NS) * STAGE;
#pragma unroll
    for (int j = 0; j < NF; ++j) f[j] = *reinterpret_cast<const v4i *>(s + (j < MI ? x_head + j * 32 * 32 : w_head + (j - MI) * 32 * 32));
  }

  // One pipeline turn after the MFMAs of step j were put in program order: the loads of step j + 5 and
  // the scheduling pattern that spreads fragment reads and loads between the MFMAs; then wait until
  // step j + 2 has landed (three newer steps may stay in flight) and a barrier makes it visible.
  template <int READS>
  __device__ __forceinline__ void turn(int j) const {
    issue(j + 5);
    constexpr int mfmas = MI * NI;
#pragma unroll
    for (int i = 0; i < mfmas; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                   // one MFMA
      if (i < READS) __builtin_amdgcn_sched_group_barrier(0x100, (READS + mfmas - 1) / mfmas, 0);  // LDS reads
    }
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(3 * P));
    __builtin_amdgcn_s_barrier();
  }

  // Integer steps [0, steps0): acc += (Lw / 8)(Lx / 8) summed over 64 elements per MFMA.
  static __device__ __forceinline__ void mfmas6(const v4i (&fh)[NF], const v2i (&ft)[NF], v16f (&acc)[MI][NI]) {
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
      for (int mi = 0; mi < MI; ++mi) {
        const v8i w = v8i{fh[MI + ni].x, fh[MI + ni].y, fh[MI + ni].z, fh[MI + ni].w, ft[MI + ni].x, ft[MI + ni].y, 0, 0};
        const v8i x = v8i{fh[mi].x, fh[mi].y, fh[mi].z, fh[mi].w, ft[mi].x, ft[mi].y, 0, 0};
        acc[mi][ni] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(w, x, acc[mi][ni], 2, 2, 0, 127, 0, 127);
      }
  }
  __device__ __forceinline__ void run_fp6(v16f (&acc)[MI][NI]) const {
    v4i h0[NF], h1[NF];
    v2i t0[NF], t1[NF];
    read6(0, h0, t0);
    for (int j = 0; j < steps0; j += 2) {
      read6(j + 1, h1, t1);
      mfmas6(h0, t0, acc);
      turn<2 * NF>(j);
      read6(j + 2, h0, t0);
      mfmas6(h1, t1, acc);
      turn<2 * NF>(j + 1);
    }
  }

  // Outlier steps [steps0, steps): acc += fp_w fp_x^T, 16 elements per MFMA.
  template <bool BF16>
  static __device__ __forceinline__ void mfmas16(const v4i (&f)[NF], v16f (&acc)[MI][NI]) {
    using Ops = FragOps<BF16 ? kBF16 : kF16>;
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
      for (int mi = 0; mi < MI; ++mi) Ops::mma(f[mi], f[MI + ni], acc[mi][ni]);
  }
  template <bool BF16>
  __device__ __forceinline__ void run_f16(v16f (&acc)[MI][NI]) const {
    v4i f0[NF], f1[NF];
    read16(steps0, f0);
    for (int j = steps0; j < steps; j += 2) {
      read16(j + 1, f1);
      mfmas16<BF16>(f0, acc);
      turn<NF>(j);
      read16(j + 2, f0);
      mfmas16<BF16>(f1, acc);
      turn<NF>(j + 1);
    }
  }

  __device__ __forceinline__ void drain() const {
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    __syncthreads();
  }
};

struct Fused6Args {
  const uint8_t *xbuf, *wbuf;  // fp6 operand buffers (activations, weights)
  const uint16_t *meta, *s_col, *w_red, *fp_x, *fp_w, *bias;
  uint16_t *out;
  int M, N, ldo, K, F;  // N: columns of this launch (wbuf, s_col, ... start at its first column)
  int n_first;          // first column of this launch inside the weight buffer's row numbering
  int N_total;          // rows of the weight buffer
};

// Per-tile vectors in LDS behind the ring: the five of TileVectors plus the two integer corrections
//   rowc[m] = 8 sum_k Lx - 64 K,  colc[n] = 8 sum_k Lw   (exact in fp32).
template <class C>
struct TileVectors6 {
  static constexpr int kBytes = (4 * C::BN + 3 * C::BM) * 4;
  float *scol, *wred, *bias, *colc, *srow, *zs, *rowc;
  __device__ __forceinline__ explicit TileVectors6(uint8_t *base) {
    scol = reinterpret_cast<float *>(base);
    wred = scol + C::BN;
    bias = wred + C::BN;
    colc = bias + C::BN;
    srow = colc + C::BN;
    zs = srow + C::BM;
    rowc = zs + C::BM;
  }
};

template <class C>
constexpr int fused6_smem() {
  return Fp6Pipe<C>::SMEM + TileVectors6<C>::kBytes;
}

template <class C, bool BF16>
__device__ __forceinline__ void fused6_tile(const Fused6Args &p, int tm, int tn, uint8_t *smem) {
  using Pipe = Fp6Pipe<C>;
  const int m0 = tm * C::BM, n0 = tn * C::BN;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;
  const Fp6Layout lx = fp6_layout(p.M, p.K), lw = fp6_layout(p.N_total, p.K);
  const TileVectors6<C> tv(smem + Pipe::SMEM);
  {
    const int32_t *xs = reinterpret_cast<const int32_t *>(p.xbuf + lx.sums_off);
    const int32_t *ws = reinterpret_cast<const int32_t *>(p.wbuf + lw.sums_off);
    for (int i = threadIdx.x; i < C::BN; i += C::kThreads) {
      const int n = n0 + i < p.N ? n0 + i : p.N - 1;
      tv.scol[i] = to_f32<BF16>(p.s_col[n]);
      tv.wred[i] = to_f32<BF16>(p.w_red[n]);
      tv.bias[i] = p.bias ? to_f32<BF16>(p.bias[n]) : 0.0f;
      tv.colc[i] = static_cast<float>(8 * ws[p.n_first + n]);
    }
    for (int i = threadIdx.x; i < C::BM; i += C::kThreads) {
      const int64_t m = m0 + i < p.M ? m0 + i : p.M - 1;
      const float s = to_f32<BF16>(p.meta[2 * m]);
      tv.srow[i] = s;
      tv.zs[i] = to_f32<BF16>(p.meta[2 * m + 1]) + 8.0f * s;
      tv.rowc[i] = static_cast<float>(8 * xs[m] - 64 * p.K);
    }
  }  // made visible by the first barrier of the pipeline

  v16f acc[C::MI][C::NI];
#pragma unroll
  for (int mi = 0; mi < C::MI; ++mi)
#pragma unroll
    for (int ni = 0; ni < C::NI; ++ni)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0.0f;

  Pipe pipe;
  const int fbytes = p.F * 2;
  pipe.init(smem, p.xbuf, lx, p.wbuf + 0, lw, m0, p.n_first + n0, p.M - m0, p.N_total - (p.n_first + n0),
            reinterpret_cast<const uint8_t *>(p.fp_x) + int64_t(m0) * fbytes,
            reinterpret_cast<const uint8_t *>(p.fp_w) + int64_t(n0) * fbytes, fbytes);
  pipe.start();
  pipe.run_fp6(acc);

  // acc = 64 S  ->  f32(integer accumulator) * (s_row * s_col), in place, one 32x32 block at a time
  float srow[C::MI], rowc[C::MI];
#pragma unroll
  for (int mi = 0; mi < C::MI; ++mi) {
    srow[mi] = tv.srow[wm * C::WM + mi * 32 + (lane & 31)];
    rowc[mi] = tv.rowc[wm * C::WM + mi * 32 + (lane & 31)];
  }
  asm volatile("s_nop 15\n\ts_nop 15");  // the last MFMA results are architecturally visible to the reads below
#pragma unroll
  for (int ni = 0; ni < C::NI; ++ni) {
    float scv[16], ccv[16];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const float4 sc = *reinterpret_cast<const float4 *>(tv.scol + wn * C::WN + ni * 32 + acc_col(g, lane));
      const float4 cc = *reinterpret_cast<const float4 *>(tv.colc + wn * C::WN + ni * 32 + acc_col(g, lane));
      scv[4 * g] = sc.x, scv[4 * g + 1] = sc.y, scv[4 * g + 2] = sc.z, scv[4 * g + 3] = sc.w;
      ccv[4 * g] = cc.x, ccv[4 * g + 1] = cc.y, ccv[4 * g + 2] = cc.z, ccv[4 * g + 3] = cc.w;
    }
#pragma unroll
    for (int mi = 0; mi < C::MI; ++mi) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const float s64 = agpr_read(acc[mi][ni][v]) * 64.0f;
        const float iacc = (s64 - rowc[mi]) - ccv[v];  // exact: integers below 2^24
        acc[mi][ni][v] = agpr_write(iacc * (srow[mi] * scv[v]));
      }
    }
  }
  pipe.template run_f16<BF16>(acc);
  pipe.drain();

  // out = storage(acc + (zs * w_red + bias)), written through the staging area
  using Store = BlockStore<C, uint16_t>;
  static_assert(Store::kBytes * C::WAVES <= Pipe::SMEM, "staging fits in the (now idle) ring");
  uint8_t *stage = smem + wave * Store::kBytes;
  const bool vec = (p.ldo & 7) == 0 && (reinterpret_cast<uintptr_t>(p.out) & 15) == 0;
  const int nw = n0 + wn * C::WN;
#pragma unroll
  for (int mi = 0; mi < C::MI; ++mi) {
    const int mb = m0 + wm * C::WM + mi * 32;
    const float zs = tv.zs[wm * C::WM + mi * 32 + (lane & 31)];
#pragma unroll
    for (int ni = 0; ni < C::NI; ++ni)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int c = wn * C::WN + ni * 32 + acc_col(g, lane);
        const float4 wr = *reinterpret_cast<const float4 *>(tv.wred + c);
        const float4 bs = *reinterpret_cast<const float4 *>(tv.bias + c);
        const uint16_t v[4] = {from_f32<BF16>(acc[mi][ni][4 * g] + (zs * wr.x + bs.x)),
                               from_f32<BF16>(acc[mi][ni][4 * g + 1] + (zs * wr.y + bs.y)),
                               from_f32<BF16>(acc[mi][ni][4 * g + 2] + (zs * wr.z + bs.z)),
                               from_f32<BF16>(acc[mi][ni][4 * g + 3] + (zs * wr.w + bs.w))};
        Store::put(stage, lane, ni, g, v);
      }
    if (mb < p.M && nw < p.N) Store::flush(stage, lane, p.out + int64_t(mb) * p.ldo + nw, p.ldo, p.M - mb, p.N - nw, vec);
    __builtin_amdgcn_sched_barrier(0);
  }
}

template <class C, bool BF16>
__global__ __launch_bounds__(C::kThreads) void gemm_fused6_kernel(Fused6Args p, int tiles_m, int tiles_n) {
  extern __shared__ __align__(16) uint8_t smem[];
  int tm, tn;
  if (!tile_of_block(blockIdx.x, tiles_m, tiles_n, tm, tn)) return;
  fused6_tile<C, BF16>(p, tm, tn, smem);
}

// One launch, two tile shapes (see gemm_i32_split_kernel).
template <class CW, class CT, bool BF16>
__global__ __launch_bounds__(CW::kThreads) void gemm_fused6_split_kernel(Fused6Args wide, Fused6Args tail,
                                                                         SplitGrid grid) {
  static_assert(CW::kThreads == CT::kThreads, "one block size");
  extern __shared__ __align__(16) uint8_t smem[];
  int tm, tn;
  const int kind = grid.locate(blockIdx.x, tm, tn);
  if (kind == 1) {
    fused6_tile<CW, BF16>(wide, tm, tn, smem);
  } else if (kind == 2) {
    fused6_tile<CT, BF16>(tail, tm, tn, smem);
  }
}

}  // namespace quik
