// int4 x int4 GEMM on the 6-bit matrix-core path of CDNA4 (gfx950), exact.
//
// v_mfma_f32_32x32x64_f8f6f4 with 6-bit E2M3 operands runs at twice the rate of the int8 MFMA.
// The E2M3 bit patterns 0 .. 15 (sign 0, exponent 00 / 01) are the uniformly spaced values
// L / 8, so a 4-bit level L = code + 8 IS an E2M3 number, zero-extended to 6 bits.  Products
// La Lw / 64 are multiples of 1/64 and their sum over K stays below 2^24 / 64 for K <= 74496 (225 K <
// 2^24), so the fp32 accumulation is exact in any order, and
//     sum_k a_k w_k = 64 S - 8 sum_k La_k - 8 sum_k Lw_k + 64 K,      S = sum_k (La_k / 8)(Lw_k / 8)
// recovers the integer accumulator exactly (every term is an integer below 2^24).  The accumulators
// start at -(8 sum_k Lw_k) / 64 (a multiple of 1/8, so still exact), and one fused multiply-add per value,
// 64 acc - (8 sum_k La_k - 64 K), finishes the job.  From there the epilogue is the one of
// gemm_kernels.h, so the output is bit-identical to the int8-MFMA path.
//
// Operand format: fp6_format.h.  Both operand buffers are stored as the sequence of LDS images the
// tiles need, so a copy instruction moves one contiguous kilobyte and every cache line is requested
// once per tile (with row-major operands a 32-byte piece per row and step asks for each line four
// times, and the 64 KB a tile touches in four steps do not survive in the 32 KB vector cache: the
// loop was bound by the cache-to-CU path at a quarter of its rate).  One MFMA k-step (64 elements)
// of a lane is a 16-byte head read plus an 8-byte tail read, both free of bank conflicts.
//
// Pipeline: a ring of 6 LDS slots, one per k-step, filled by global_load_lds_dwordx4.  While step j
// feeds the MFMAs, the fragments of step j + 1 are read into registers and steps j + 2 .. j + 5 are
// landing (the slot of step j was handed to step j + 6 when step j's reads were done); the outlier
// GEMM's fp16/bf16 steps (16 elements each, 32 bytes per row like a head) run through the same ring
// after the integer steps.
#pragma once
#include "fp6_format.h"
#include "gemm_kernels.h"

namespace quik {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v8i __attribute__((ext_vector_type(8)));

// One wave-wide copy global -> LDS (see dma_load16) whose instruction offset moves both addresses: the three
// kilobytes of a block unit are copied with one source pointer and one LDS base.
// (Hazards: one wait state between the scalar write of m0 and the copy that reads it, the s_nop 0; m0 is in the
// clobber list, so the compiler does not keep a value of its own in it across the statement; the "memory" clobber
// keeps LDS accesses of the compiler on their side of the copy, and completion is awaited through vmcnt.)
template <int OFFSET>
__device__ __forceinline__ void dma_load16k(const uint8_t *sbase, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 offset:%3"
               : : "s"(lds_addr), "v"(voff), "s"(sbase), "n"(OFFSET) : "memory", "m0");
}

template <class C>
struct Fp6Pipe {
  static constexpr int MI = C::MI, NI = C::NI, NS = 6, NF = MI + NI;
  // a wave's fragments start at a 64-row block of the operand, or the wave has a single 32-row fragment (then it may
  // be the second half of a block)
  static_assert(C::WM % 64 == 0 || C::MI == 1, "a wave's token rows");
  static_assert(C::WN % 64 == 0 || C::NI == 1, "a wave's weight rows");
  static_assert(C::WAVES == 4 || C::WAVES == 8, "copy assignment below");
  // LDS slot of one step: the 3 KB units of the tile's X blocks, then of its W blocks, as they are in memory
  static constexpr int W_OFF = C::BM * 48;
  static constexpr int STAGE = (C::BM + C::BN) * 48;
  static constexpr int SMEM = NS * STAGE;
  // Copies per step: 3 per 64-row block (head image of rows 0..31, of rows 32..63, tail image), XB + WB blocks.
  // Every wave copies one whole block from its source A (X block w, or W block w - XB when the tile has
  // fewer than 4 X blocks), and NB further kilobytes from its source B:
  //   256x256: W block w (3);  256x128: W block w % 2, pieces w / 2 and w / 2 + 1 (piece 1 is copied twice);
  //   128x128: none;  128x64: none (two waves copy the one W block: the same bytes to the same place).
  static constexpr int XB = C::BM / 64, WB = C::BN / 64;
  // (eight waves, 256x256: one block per wave, no source B)
  static constexpr int NB = C::WAVES == 8 ? 0 : XB + WB == 8 ? 3 : XB + WB == 6 ? 2 : 0;
  static_assert((XB == 4 && (WB == 4 || WB == 2)) || (XB == 2 && (WB == 2 || WB == 1)), "supported tile shapes");
  static_assert(C::WAVES == 4 || XB + WB == 8, "eight waves copy eight blocks");
  static constexpr int P = 3 + NB;  // copies per wave and step
  static_assert(3 * P <= 63, "three steps in flight must fit the vmcnt counter");

  uint8_t *smem;
  uint32_t lds0;
  const uint8_t *pa, *pb;   // wave-uniform: sources of the next step to be copied
  uint32_t da, db;          // wave-uniform: destinations inside a slot
  uint32_t fill;            // wave-uniform: LDS address of the slot the next copy fills
  int left;                 // steps whose copy has not been issued yet
  uint32_t lane16;
  uint32_t rd;              // byte offset of the slot the next fragment read looks at
  int steps0, steps;        // integer steps, all steps
  uint32_t x_head, w_head;  // this lane's head offsets inside a slot (fragment j: + 1024 j)
  uint32_t x_head3[3], w_head3[3], tail3[3][NF];  // the same offsets inside slots 0, 2 and 4 (for steps whose slot is
                                                  // known at compile time: the odd slot is an immediate offset away)
  uint32_t tail[NF];        // this lane's tail offsets inside a slot, one register per fragment: reads that share
                            // a base register are paired into one 4-register read by the compiler, and the halves
                            // then have to be copied into the operand tuples behind an exposed LDS round trip

  // xb0 / wb0: first 64-row block of the tile in each operand buffer
  // unit0: first unit (step) of every block to copy; n_int / n_f: integer and outlier steps from there on
  // (-1: all of the block's, from its first unit)
  __device__ __forceinline__ void init(uint8_t *smem_, const uint8_t *xbuf, const Fp6Layout &lx, int64_t xb0,
                                       const uint8_t *wbuf, const Fp6Layout &lw, int64_t wb0, int unit0 = 0,
                                       int n_int = -1, int n_f = -1) {
    smem = smem_;
    lds0 = lds_address(smem_);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;
    auto block_ptr = [&](bool is_x, int blk) {
      const Fp6Layout &l = is_x ? lx : lw;
      int64_t B = (is_x ? xb0 : wb0) + blk;
      B = B < l.blocks ? B : l.blocks - 1;  // blocks past the matrix: any valid block, results never stored
      return (is_x ? xbuf : wbuf) + B * l.block_bytes + int64_t(unit0) * 3072;
    };
    {
      const bool is_x = wave < XB;
      const int blk = is_x ? wave : (wave - XB) % WB;
      pa = block_ptr(is_x, blk);
      da = (is_x ? 0 : W_OFF) + blk * 3072;
    }
    pb = pa;
    db = da;
    if constexpr (NB == 3) {
      pb = block_ptr(false, wave);
      db = W_OFF + wave * 3072;
    } else if constexpr (NB == 2) {
      pb = block_ptr(false, wave & 1) + (wave >> 1) * 1024;
      db = W_OFF + (wave & 1) * 3072 + (wave >> 1) * 1024;
    }
    lane16 = lane * 16;
    fill = lds0;
    rd = 0;
    steps0 = n_int < 0 ? static_cast<int>(lx.steps) : n_int;
    steps = steps0 + (n_f < 0 ? static_cast<int>(lx.fsteps) : n_f);
    left = steps;
    const int r = lane & 31, h = lane >> 5;
    const int slot16 = (h ^ ((r >> 3) & 1)) << 4;
    // first 32-row fragment of the wave in each operand: block fx0 / 2 (fw0 / 2), half fx0 % 2 (odd only for waves of
    // a single fragment)
    const int fx0 = wm * C::WM / 32, fw0 = wn * C::WN / 32;
    x_head = (fx0 >> 1) * 3072 + (fx0 & 1) * 1024 + r * 32 + slot16;
    w_head = W_OFF + (fw0 >> 1) * 3072 + (fw0 & 1) * 1024 + r * 32 + slot16;
#pragma unroll
    for (int j = 0; j < NF; ++j) {
      const int jj = j < MI ? j : j - MI;
      const int f0 = j < MI ? fx0 : fw0;
      tail[j] = (j < MI ? 0 : W_OFF) + (f0 >> 1) * 3072 + (jj >> 1) * 3072 + 2048 + h * 512 +
                ((((f0 & 1) + jj) & 1) * 32 + r) * 8;
      asm volatile("" : "+v"(tail[j]));  // unrelated values as far as the compiler can tell (empty statement: no hazard)
    }
#pragma unroll
    for (int q = 0; q < 3; ++q) {
      x_head3[q] = x_head + q * 2 * STAGE;
      w_head3[q] = w_head + q * 2 * STAGE;
#pragma unroll
      for (int j = 0; j < NF; ++j) {
        tail3[q][j] = tail[j] + q * 2 * STAGE;
        asm volatile("" : "+v"(tail3[q][j]));
      }
    }
  }

  // Copy G (0 .. P-1) of the step being copied; after the last one the scalar bookkeeping: two pointer
  // bumps and one slot bump.  Past the last step the pointers stop and the last step is copied again into
  // a slot nobody reads.
  // FS: slot being filled when known at compile time (the caller keeps `fill` consistent), -1: `fill`
  template <int G, int FS = -1>
  __device__ __forceinline__ void issue_one() {
    const uint32_t slot = FS < 0 ? fill : lds0 + (FS < 0 ? 0 : FS) * STAGE;
    if constexpr (G < 3) {
      dma_load16k<G * 1024>(pa, lane16, slot + da);
    } else {
      dma_load16k<(G - 3) * 1024>(pb, lane16, slot + db);
    }
    if constexpr (G == P - 1) {
      const int adv = left > 1 ? 3072 : 0;
      left -= 1;
      pa += adv;
      pb += adv;
      if constexpr (FS < 0) {
        fill += STAGE;
        fill = fill == lds0 + NS * STAGE ? lds0 : fill;
      }
    }
  }
  template <int G = 0>
  __device__ __forceinline__ void issue() {
    if constexpr (G < P) {
      issue_one<G>();
      issue<G + 1>();
    }
  }

  // Fill the ring: afterwards steps 0 and 1 are visible and steps 2 .. 4 are in flight; the copies of step 5
  // are made during the MFMAs of step 0.
  __device__ __forceinline__ void start() {
    issue();
    issue();
    issue();
    issue();
    issue();
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(3 * P));
    __syncthreads();
  }

  __device__ __forceinline__ void next_read_slot() {
    rd += STAGE;
    rd = rd == NS * STAGE ? 0 : rd;
  }
  __device__ __forceinline__ void previous_read_slot() { rd = rd == 0 ? (NS - 1) * STAGE : rd - STAGE; }

  // fragment j (32 rows) of this wave: head image j, tail image j / 2 at row offset 32 (j % 2)
  // RS: slot being read when known at compile time, -1: `rd`
  template <int J, int RS = -1>
  __device__ __forceinline__ void read6_one(v4i (&fh)[NF], v2i (&ft)[NF]) const {
    constexpr int jj = J < MI ? J : J - MI;
    if constexpr (RS < 0) {
      const uint8_t *s = smem + rd;
      fh[J] = *reinterpret_cast<const v4i *>(s + (J < MI ? x_head : w_head) + (jj >> 1) * 3072 + (jj & 1) * 1024);
      ft[J] = *reinterpret_cast<const v2i *>(s + tail[J]);
    } else {
      constexpr int q = (RS < 0 ? 0 : RS) / 2, odd = ((RS < 0 ? 0 : RS) % 2) * STAGE;
      fh[J] = *reinterpret_cast<const v4i *>(smem + (J < MI ? x_head3[q] : w_head3[q]) + odd + (jj >> 1) * 3072 +
                                             (jj & 1) * 1024);
      ft[J] = *reinterpret_cast<const v2i *>(smem + tail3[q][J] + odd);
    }
  }
  template <int J>
  __device__ __forceinline__ void read16_one(v4i (&f)[NF]) const {
    constexpr int jj = J < MI ? J : J - MI;
    f[J] = *reinterpret_cast<const v4i *>(smem + rd + (J < MI ? x_head : w_head) + (jj >> 1) * 3072 + (jj & 1) * 1024);
  }
  template <int J = 0>
  __device__ __forceinline__ void read6(v4i (&fh)[NF], v2i (&ft)[NF]) {
    if constexpr (J < NF) {
      read6_one<J>(fh, ft);
      read6<J + 1>(fh, ft);
    } else {
      next_read_slot();
    }
  }
  template <int J = 0>
  __device__ __forceinline__ void read16(v4i (&f)[NF]) {
    if constexpr (J < NF) {
      read16_one<J>(f);
      read16<J + 1>(f);
    } else {
      next_read_slot();
    }
  }

  // MFMA I (0 .. MI NI - 1) of a step: block (mi, ni) = (I % MI, I / MI)
  template <int I>
  static __device__ __forceinline__ void mfma6_one(const v4i (&fh)[NF], const v2i (&ft)[NF], v16f (&acc)[MI][NI]) {
    constexpr int mi = I % MI, ni = I / MI;
    const v8i w = v8i{fh[MI + ni].x, fh[MI + ni].y, fh[MI + ni].z, fh[MI + ni].w, ft[MI + ni].x, ft[MI + ni].y, 0, 0};
    const v8i x = v8i{fh[mi].x, fh[mi].y, fh[mi].z, fh[mi].w, ft[mi].x, ft[mi].y, 0, 0};
    // Block scales of 2^0.  Written as scale operands 0, 0 the compiler emits the plain v_mfma_f32_32x32x64_f8f6f4,
    // whose scales are 1.0 by definition; with the equivalent E8M0 value 127 spelled out it emits the scaled form,
    // a scale-load instruction in front of every MFMA, which costs an issue slot each (measured on chains of
    // dependent MFMAs: identical results, 21 % more time).  Were a compiler to keep the scaled form WITH operands 0,
    // every product would be scaled by 2^-127: the Makefile's check-mfma target reads the mnemonics of the built
    // object and fails the build on a scaled f8f6f4 MFMA.
    acc[mi][ni] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(w, x, acc[mi][ni], 2, 2, 0, 0, 0, 0);
  }
  template <bool BF16, int I>
  static __device__ __forceinline__ void mfma16_one(const v4i (&f)[NF], v16f (&acc)[MI][NI]) {
    constexpr int mi = I % MI, ni = I / MI;
    FragOps<BF16 ? kBF16 : kF16>::mma(f[mi], f[MI + ni], acc[mi][ni]);
  }

  // One step, cut into P chunks: chunk G holds its share of the step's MFMAs (on the fragments in `cur`),
  // of the next step's fragment reads (into `nxt`) and one of the P copies of the step five ahead of the
  // one in the MFMAs.  A copy instruction occupies the wave until the memory pipeline has taken its 64
  // addresses; six of them in a row at the start of a step stall the MFMA issue for as long as the copies
  // take, so they go one by one between groups of MFMAs.  Then: wait until the step after next has
  // landed (the three newer ones stay in flight) and a barrier makes it visible; behind it every wave has
  // issued the MFMAs of this step, which waited for their fragments, so this step's slot may be overwritten
  // by the copies issued during the next step.
  // RS / FS: the slots read and filled during this step when they are known at compile time (six steps in a
  // row return to the same slots, so `rd` and `fill` stay valid without being touched), -1: `rd` / `fill`
  template <int RS = -1, int FS = -1, int G = 0>
  __device__ __forceinline__ void step6(const v4i (&ch)[NF], const v2i (&ct)[NF], v4i (&nh)[NF], v2i (&nt)[NF],
                                        v16f (&acc)[MI][NI]) {
    constexpr int MM = MI * NI;
    if constexpr (G < P) {
      constexpr int r_lo = G * NF / P, r_hi = (G + 1) * NF / P, m_lo = G * MM / P, m_hi = (G + 1) * MM / P;
      chunk_reads6<RS, r_lo, r_hi>(nh, nt);
      chunk_mfmas6<m_lo, m_hi>(ch, ct, acc);
      if constexpr (m_hi > m_lo) {
#pragma unroll
        for (int i = m_lo; i < m_hi; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, (2 * (r_hi - r_lo) + (m_hi - m_lo) - 1) / (m_hi - m_lo), 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      issue_one<G, FS>();
      __builtin_amdgcn_sched_barrier(0);
      step6<RS, FS, G + 1>(ch, ct, nh, nt, acc);
    } else {
      if constexpr (RS < 0) next_read_slot();
      __builtin_amdgcn_s_waitcnt(vmcnt_imm(3 * P));
      __builtin_amdgcn_s_barrier();
    }
  }
  template <int RS, int LO, int HI>
  __device__ __forceinline__ void chunk_reads6(v4i (&nh)[NF], v2i (&nt)[NF]) const {
    if constexpr (LO < HI) {
      read6_one<LO, RS>(nh, nt);
      chunk_reads6<RS, LO + 1, HI>(nh, nt);
    }
  }
  template <int LO, int HI>
  static __device__ __forceinline__ void chunk_mfmas6(const v4i (&ch)[NF], const v2i (&ct)[NF], v16f (&acc)[MI][NI]) {
    if constexpr (LO < HI) {
      mfma6_one<LO>(ch, ct, acc);
      chunk_mfmas6<LO + 1, HI>(ch, ct, acc);
    }
  }
  template <bool BF16, int G = 0>
  __device__ __forceinline__ void step16(const v4i (&cf)[NF], v4i (&nf)[NF], v16f (&acc)[MI][NI]) {
    constexpr int MM = MI * NI;
    if constexpr (G < P) {
      constexpr int r_lo = G * NF / P, r_hi = (G + 1) * NF / P, m_lo = G * MM / P, m_hi = (G + 1) * MM / P;
      chunk_reads16<r_lo, r_hi>(nf);
      chunk_mfmas16<BF16, m_lo, m_hi>(cf, acc);
      if constexpr (m_hi > m_lo) {
#pragma unroll
        for (int i = m_lo; i < m_hi; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, ((r_hi - r_lo) + (m_hi - m_lo) - 1) / (m_hi - m_lo), 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      issue_one<G>();
      __builtin_amdgcn_sched_barrier(0);
      step16<BF16, G + 1>(cf, nf, acc);
    } else {
      next_read_slot();
      __builtin_amdgcn_s_waitcnt(vmcnt_imm(3 * P));
      __builtin_amdgcn_s_barrier();
    }
  }
  template <int LO, int HI>
  __device__ __forceinline__ void chunk_reads16(v4i (&nf)[NF]) const {
    if constexpr (LO < HI) {
      read16_one<LO>(nf);
      chunk_reads16<LO + 1, HI>(nf);
    }
  }
  template <bool BF16, int LO, int HI>
  static __device__ __forceinline__ void chunk_mfmas16(const v4i (&cf)[NF], v16f (&acc)[MI][NI]) {
    if constexpr (LO < HI) {
      mfma16_one<BF16, LO>(cf, acc);
      chunk_mfmas16<BF16, LO + 1, HI>(cf, acc);
    }
  }

  // Integer steps [0, steps0): acc += (Lw / 8)(Lx / 8) summed over 64 elements per MFMA.
  __device__ __forceinline__ void run_fp6(v16f (&acc)[MI][NI]) {
    v4i h0[NF], h1[NF];
    v2i t0[NF], t1[NF];
    read6(h0, t0);
    // here: step 0 in h0 / t0, `rd` at slot 1, `fill` at slot 5.  Six steps at a time with the slots as
    // immediates (no address arithmetic in the loop), then the remaining pairs with `rd` / `fill`
    int j = 0;
    for (; j + 6 <= steps0; j += 6) {
      step6<1, 5>(h0, t0, h1, t1, acc);
      step6<2, 0>(h1, t1, h0, t0, acc);
      step6<3, 1>(h0, t0, h1, t1, acc);
      step6<4, 2>(h1, t1, h0, t0, acc);
      step6<5, 3>(h0, t0, h1, t1, acc);
      step6<0, 4>(h1, t1, h0, t0, acc);
    }
    for (; j < steps0; j += 2) {
      step6(h0, t0, h1, t1, acc);
      step6(h1, t1, h0, t0, acc);
    }
    previous_read_slot();  // the last read looked at the first outlier step (or a dead slot) as 6-bit data
  }

  // Outlier steps [steps0, steps): acc += fp_w fp_x^T, 16 elements per MFMA.
  template <bool BF16>
  __device__ __forceinline__ void run_f16(v16f (&acc)[MI][NI]) {
    v4i f0[NF], f1[NF];
    read16(f0);
    for (int j = steps0; j < steps; j += 2) {
      step16<BF16>(f0, f1, acc);
      step16<BF16>(f1, f0, acc);
    }
  }

  __device__ __forceinline__ void drain() const {
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    __syncthreads();
  }
};

struct Fused6Args {
  const uint8_t *xbuf, *wbuf;  // operand buffers (activations, weights), outlier columns included
  const uint16_t *meta, *s_col, *w_red, *bias;
  uint16_t *out;
  int M, N, ldo, K, F;  // N: columns of this launch (wbuf, s_col, ... start at its first column)
  int n_first;          // first column of this launch inside the weight buffer's row numbering
  int N_total;          // rows of the weight buffer
};

// Per-tile vectors in LDS behind the ring: the five of TileVectors plus the two integer corrections
//   rowc[m] = 8 sum_k Lx - 64 K,  colc[n] = -(8 sum_k Lw) / 64 (the accumulators' start value)   (exact in fp32).
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

// Split over K (few tiles, long K): `splits` workgroups per tile take `per` integer steps each and add their raw
// accumulators (int32, or the exact fp32 sums of the 6-bit path) through `partials`; the one that arrives last (counted in `counters`, which are zero between
// launches) sums them, exactly, and goes on with the outlier steps and the epilogue as a whole-K tile would: the
// result has the same bits.  partials: [tile][split][register][thread], 4 bytes each.
struct SplitK {
  int splits, per, grid_tiles;
  uint32_t *counters;
  int32_t *partials;
};
// The partial sums cross from one XCD's L2 to another's.  A device-wide fence would do that by writing back and
// invalidating the whole L2 of the XCD, once per wave, under the operand streams of the other tiles (measured: the
// launch takes three times as long), and device-scope atomic loads are issued one at a time.  Instead the partial
// sums are moved by ordinary 16-byte stores and loads that carry the device-scope cache policy (sc1: past the L2,
// one access at a time); the stores are complete (vmcnt) before the workgroup's barrier and the arrival count
// behind it, and the loads are issued only after the count has been seen.
// partials: [tile][split][group of 4 registers][thread][4].
// (the wait states: a store of more than 8 bytes reads its data registers over several cycles, and the instruction
// after this statement may be one that overwrites them; between the compiler's own instructions the compiler
// keeps that distance, around inline assembly it does not)
__device__ __forceinline__ void splitk_store4(int32_t *p, v4i v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 2" : : "v"(p), "v"(v) : "memory");
}
// (a wait only: no register or wait-state hazard; "memory" keeps the compiler from moving stores across it)
__device__ __forceinline__ void splitk_stores_done() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
// eight 16-byte loads, STRIDE int32 apart, and the wait for them in one statement: the compiler sees the
// registers only once they hold the data (hazards: the outputs are early-clobber, so no load's destination
// overlaps an address register that a later load of the statement still reads; the statement ends with
// vmcnt(0), so nothing it started is in flight when the compiler's instructions resume)
template <int STRIDE>
__device__ __forceinline__ void splitk_load8(const int32_t *p, v4i *r) {
  asm volatile(
      "global_load_dwordx4 %0, %8, off sc1\n\tglobal_load_dwordx4 %1, %9, off sc1\n\t"
      "global_load_dwordx4 %2, %10, off sc1\n\tglobal_load_dwordx4 %3, %11, off sc1\n\t"
      "global_load_dwordx4 %4, %12, off sc1\n\tglobal_load_dwordx4 %5, %13, off sc1\n\t"
      "global_load_dwordx4 %6, %14, off sc1\n\tglobal_load_dwordx4 %7, %15, off sc1\n\t"
      "s_waitcnt vmcnt(0)"
      : "=&v"(r[0]), "=&v"(r[1]), "=&v"(r[2]), "=&v"(r[3]), "=&v"(r[4]), "=&v"(r[5]), "=&v"(r[6]), "=&v"(r[7])
      : "v"(p), "v"(p + STRIDE), "v"(p + 2 * STRIDE), "v"(p + 3 * STRIDE), "v"(p + 4 * STRIDE), "v"(p + 5 * STRIDE),
        "v"(p + 6 * STRIDE), "v"(p + 7 * STRIDE)
      : "memory");
}

// Adds a tile's raw accumulators over the splits (see SplitK).  Returns false in every workgroup but the one that
// arrived last; there `acc` holds the whole-K sums (INT: int32 bit patterns, else fp32) and the ring is idle.
template <class C, bool INT>
__device__ __forceinline__ bool splitk_combine(v16f (&acc)[C::MI][C::NI], const SplitK &sk, int tile_id, int split,
                                               uint8_t *smem) {
  static_assert(C::MI * C::NI == 4, "16 groups of 4 registers");
  constexpr int STRIDE = C::kThreads * 4;
  asm volatile("s_nop 15\n\ts_nop 15");  // the last MFMA results are architecturally visible
  int32_t *mine = sk.partials + (int64_t(tile_id) * sk.splits + split) * 16 * STRIDE + threadIdx.x * 4;
#pragma unroll
  for (int b = 0; b < C::MI * C::NI; ++b)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const v16f &a = acc[b / C::NI][b % C::NI];
      splitk_store4(mine + (b * 4 + g) * STRIDE,
                    v4i{__float_as_int(agpr_read(a[4 * g])), __float_as_int(agpr_read(a[4 * g + 1])),
                        __float_as_int(agpr_read(a[4 * g + 2])), __float_as_int(agpr_read(a[4 * g + 3]))});
    }
  splitk_stores_done();
  __syncthreads();
  int *last_s = reinterpret_cast<int *>(smem);
  if (threadIdx.x == 0) {
    const uint32_t before = __hip_atomic_fetch_add(sk.counters + tile_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *last_s = before == static_cast<uint32_t>(sk.splits - 1);
  }
  __syncthreads();
  const bool last = *last_s != 0;
  __syncthreads();
  if (!last) return false;
  for (int q = 0; q < sk.splits; ++q) {  // exact sums: the order does not matter
    if (q == split) continue;
    const int32_t *theirs = sk.partials + (int64_t(tile_id) * sk.splits + q) * 16 * STRIDE + threadIdx.x * 4;
    v4i t[16];
    splitk_load8<STRIDE>(theirs, t);
    splitk_load8<STRIDE>(theirs + 8 * STRIDE, t + 8);
#pragma unroll
    for (int b = 0; b < C::MI * C::NI; ++b)
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v16f &a = acc[b / C::NI][b % C::NI];
          const float mine_v = agpr_read(a[4 * g + e]);
          a[4 * g + e] = agpr_write(INT ? __int_as_float(__float_as_int(mine_v) + t[b * 4 + g][e])
                                        : mine_v + __int_as_float(t[b * 4 + g][e]));
        }
  }
  if (threadIdx.x == 0) __hip_atomic_store(sk.counters + tile_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return true;
}

template <class C, bool BF16, bool SPLITK = false>
__device__ __forceinline__ void fused6_tile(const Fused6Args &p, int tm, int tn, uint8_t *smem, int split = 0,
                                            int tile_id = 0, const SplitK *sk = nullptr) {
  using Pipe = Fp6Pipe<C>;
  const int m0 = tm * C::BM, n0 = tn * C::BN;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;
  const Fp6Layout lx = fp6_layout(p.M, p.K, p.F), lw = fp6_layout(p.N_total, p.K, p.F);
  const TileVectors6<C> tv(smem + Pipe::SMEM);
  {
    const int32_t *xs = reinterpret_cast<const int32_t *>(p.xbuf + lx.sums_off);
    const int32_t *ws = reinterpret_cast<const int32_t *>(p.wbuf + lw.sums_off);
    for (int i = threadIdx.x; i < C::BN; i += C::kThreads) {
      const int n = n0 + i < p.N ? n0 + i : p.N - 1;
      tv.scol[i] = to_f32<BF16>(p.s_col[n]);
      tv.wred[i] = p.w_red ? to_f32<BF16>(p.w_red[n]) : 0.0f;
      tv.bias[i] = p.bias ? to_f32<BF16>(p.bias[n]) : 0.0f;
      tv.colc[i] = static_cast<float>(ws[p.n_first + n]) * -0.125f;
    }
    for (int i = threadIdx.x; i < C::BM; i += C::kThreads) {
      const int64_t m = m0 + i < p.M ? m0 + i : p.M - 1;
      // asymmetric: meta holds (scale, zero) pairs; symmetric (no w_red): one scale per row and no zero term
      const float s = to_f32<BF16>(p.meta[p.w_red ? 2 * m : m]);
      tv.srow[i] = s;
      tv.zs[i] = p.w_red ? to_f32<BF16>(p.meta[2 * m + 1]) + 8.0f * s : 0.0f;
      tv.rowc[i] = static_cast<float>(8 * xs[m] - 64 * p.K);
    }
  }  // made visible by the first barrier of the pipeline

  Pipe pipe;
  const int total = static_cast<int>(lx.steps);
  int k0 = 0, k1 = total;
  if constexpr (SPLITK) {
    k0 = split * sk->per;
    k1 = k0 + sk->per < total ? k0 + sk->per : total;
    pipe.init(smem, p.xbuf, lx, m0 / 64, p.wbuf, lw, (p.n_first + n0) / 64, k0, k1 - k0, 0);
  } else {
    pipe.init(smem, p.xbuf, lx, m0 / 64, p.wbuf, lw, (p.n_first + n0) / 64);
  }
  pipe.start();  // its barrier also makes the vectors visible

  v16f acc[C::MI][C::NI];
#pragma unroll
  for (int ni = 0; ni < C::NI; ++ni)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      float4 cc = *reinterpret_cast<const float4 *>(tv.colc + wn * C::WN + ni * 32 + acc_col(g, lane));
      if (SPLITK && split != 0) cc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);  // the column term enters once
#pragma unroll
      for (int mi = 0; mi < C::MI; ++mi)
        acc[mi][ni][4 * g] = cc.x, acc[mi][ni][4 * g + 1] = cc.y, acc[mi][ni][4 * g + 2] = cc.z, acc[mi][ni][4 * g + 3] = cc.w;
    }
  pipe.run_fp6(acc);
  if constexpr (SPLITK) {
    pipe.drain();  // the copies past the last step have landed too: the ring is free
    if (!splitk_combine<C, false>(acc, *sk, tile_id, split, smem)) return;
    if (lx.fsteps > 0) {
      pipe.init(smem, p.xbuf, lx, m0 / 64, p.wbuf, lw, (p.n_first + n0) / 64, total, 0, static_cast<int>(lx.fsteps));
      pipe.start();
    } else {
      pipe.steps0 = pipe.steps = 0;
    }
  }

  // acc = S - colc / 64  ->  f32(integer accumulator) * (s_row * s_col) + (zs * w_red + bias), in place, one 32x32
  // block at a time.  The zero-point and bias term goes in here, as the addend of the multiply that is needed anyway:
  // the epilogue then only converts and stores (one instruction per value less than adding it there).
  float srow[C::MI], rowc[C::MI], zsr[C::MI];
#pragma unroll
  for (int mi = 0; mi < C::MI; ++mi) {
    srow[mi] = tv.srow[wm * C::WM + mi * 32 + (lane & 31)];
    rowc[mi] = tv.rowc[wm * C::WM + mi * 32 + (lane & 31)];
    zsr[mi] = tv.zs[wm * C::WM + mi * 32 + (lane & 31)];
  }
  asm volatile("s_nop 15\n\ts_nop 15");  // the last MFMA results are architecturally visible to the reads below
#pragma unroll
  for (int ni = 0; ni < C::NI; ++ni) {
    float scv[16], wrv[16], bsv[16];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int c = wn * C::WN + ni * 32 + acc_col(g, lane);
      const float4 sc = *reinterpret_cast<const float4 *>(tv.scol + c);
      const float4 wr = *reinterpret_cast<const float4 *>(tv.wred + c);
      const float4 bs = *reinterpret_cast<const float4 *>(tv.bias + c);
      scv[4 * g] = sc.x, scv[4 * g + 1] = sc.y, scv[4 * g + 2] = sc.z, scv[4 * g + 3] = sc.w;
      wrv[4 * g] = wr.x, wrv[4 * g + 1] = wr.y, wrv[4 * g + 2] = wr.z, wrv[4 * g + 3] = wr.w;
      bsv[4 * g] = bs.x, bsv[4 * g + 1] = bs.y, bsv[4 * g + 2] = bs.z, bsv[4 * g + 3] = bs.w;
    }
#pragma unroll
    for (int mi = 0; mi < C::MI; ++mi) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const float iacc = __builtin_fmaf(agpr_read(acc[mi][ni][v]), 64.0f, -rowc[mi]);  // exact: integers below 2^24
        acc[mi][ni][v] = agpr_write(__builtin_fmaf(iacc, srow[mi] * scv[v], __builtin_fmaf(zsr[mi], wrv[v], bsv[v])));
      }
    }
  }
  pipe.template run_f16<BF16>(acc);
  pipe.drain();

  // out = storage(acc), written through a staging area in the (now idle) ring: all MI row
  // blocks of the wave are staged, then read back as whole row segments, then stored, so the LDS round trip and
  // the store issue are paid once per tile and not once per row block.  The per-column vectors are read once;
  // the fragment registers are free by now.
  using Store = BlockStore<C, uint16_t>;
  static_assert(Store::kBytes * C::MI * C::WAVES <= Pipe::SMEM, "staging fits in the ring");
  uint8_t *stage = smem + wave * (Store::kBytes * C::MI);
  const bool vec = (p.ldo & 7) == 0 && (reinterpret_cast<uintptr_t>(p.out) & 15) == 0;
  const int nw = n0 + wn * C::WN, mw = m0 + wm * C::WM;
#pragma unroll
  for (int mi = 0; mi < C::MI; ++mi)
#pragma unroll
    for (int ni = 0; ni < C::NI; ++ni)
#pragma unroll
      for (int g = 0; g < 4; ++g)
        Store::put_pairs(stage + mi * Store::kBytes, lane, ni, g,
                         pack2_from_f32<BF16>(acc[mi][ni][4 * g], acc[mi][ni][4 * g + 1]),
                         pack2_from_f32<BF16>(acc[mi][ni][4 * g + 2], acc[mi][ni][4 * g + 3]));
  if (vec && p.M - mw >= C::WM && p.N - nw >= C::WN) {  // interior (wave-uniform): straight-line code
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    v4i piece[C::MI][Store::kIters];
#pragma unroll
    for (int mi = 0; mi < C::MI; ++mi) Store::read_block(stage + mi * Store::kBytes, lane, piece[mi]);
#pragma unroll
    for (int mi = 0; mi < C::MI; ++mi)
      Store::write_block(piece[mi], lane, p.out + int64_t(mw + mi * 32) * p.ldo + nw, p.ldo);
  } else {
#pragma unroll
    for (int mi = 0; mi < C::MI; ++mi) {
      const int mb = mw + mi * 32;
      if (mb < p.M && nw < p.N)
        Store::flush(stage + mi * Store::kBytes, lane, p.out + int64_t(mb) * p.ldo + nw, p.ldo, p.M - mb, p.N - nw, vec);
    }
  }
}

template <class C, bool BF16>
__global__ __launch_bounds__(C::kThreads) void gemm_fused6_kernel(Fused6Args p, int tiles_m, int tiles_n) {
  extern __shared__ __align__(16) uint8_t smem[];
  int tm, tn;
  if (!tile_of_block(blockIdx.x, tiles_m, tiles_n, tm, tn)) return;
  fused6_tile<C, BF16>(p, tm, tn, smem);
}

// K split over sk.splits workgroups per tile: block b works on tile b % grid_tiles, split b / grid_tiles.
template <class C, bool BF16>
__global__ __launch_bounds__(C::kThreads) void gemm_fused6_splitk_kernel(Fused6Args p, int tiles_m, int tiles_n,
                                                                          SplitK sk) {
  extern __shared__ __align__(16) uint8_t smem[];
  int tm, tn;
  const int split = blockIdx.x / sk.grid_tiles;
  if (!tile_of_block(blockIdx.x - split * sk.grid_tiles, tiles_m, tiles_n, tm, tn)) return;
  fused6_tile<C, BF16, true>(p, tm, tn, smem, split, tm * tiles_n + tn, &sk);
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
