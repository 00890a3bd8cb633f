// Integer GEMMs of the MixedQLinear forward path on CDNA4 (gfx950) matrix cores:
//   int4 x int4 -> int32, int8 x int8 -> int32 (the unfused ops), and the fused forward
//   out = dtype( f32(acc) * (s_row * s_col) + (zero + 2^(bits-1) s_row) * w_red + fp_x fp_w^T + bias ).
//
// Operands are "TN": X [M, K] (activations) and W [N, K] (weights) are both K-contiguous, the
// native operand order of v_mfma_i32_32x32x32_i8: lane l supplies 16 consecutive K bytes of row
// l % 32, K half l / 32.  X and W fragments are fetched with the same lane -> K mapping, so any
// permutation of K inside one instruction is harmless; the int4 path exploits that:
//   a packed dword w holds nibbles n0..n7;  lo = (w << 4) & 0xF0F0F0F0 is int8x4 {16 n0, 16 n2,
//   16 n4, 16 n6},  hi = w & 0xF0F0F0F0 is {16 n1, 16 n3, 16 n5, 16 n7}.  Both operands are
//   unpacked the same way, products come out 256x too large, and the exact accumulator is
//   recovered with an arithmetic shift by 8 (needs 16384 K < 2^31, i.e. K < 131072).
// There is no int4 MFMA on CDNA4; int4 saves HBM and LDS bytes only.
//
// The weight fragment is passed as the MFMA's first (row) operand and the activation fragment
// as the second (column) operand.  A lane then owns, per 32x32 block, one token row m = l % 32
// and four consecutive output columns n per register group, which makes the epilogue's stores
// 16-byte (int32) or 8-byte (fp16) vectors and its per-column vectors contiguous loads.
//
// One workgroup computes a BM x BN tile with WAVES_M x WAVES_N wavefronts, each wave a
// (BM/WAVES_M) x (BN/WAVES_N) sub-tile of 32x32 blocks held in accumulator registers.  Two main
// loops exist: a plain double-buffered one that accepts any shape (ragged K, tiny tiles), and
// the direct-to-LDS software-pipelined one used for the large tiles (see mainloop_dma).
// Workgroup ids are remapped so that the ids that land on one XCD (id % 8) cover neighbouring
// tiles and share their L2.
#pragma once
#include <type_traits>

#include "common.h"

namespace quik {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

enum Mode { kInt4 = 0, kInt8 = 1, kF16 = 2, kBF16 = 3 };

template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, int PIPE_ = 0>
struct Cfg {
  static constexpr int BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
  static constexpr int BKB = 64;        // K bytes per row and stage
  static constexpr int PIPE = PIPE_;    // 0: plain double buffer, 2: direct-to-LDS 4-stage ring
  static constexpr int WAVES = WAVES_M * WAVES_N;
  static constexpr int kThreads = WAVES * 64;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int MI = WM / 32, NI = WN / 32;
  // plain loop: rows padded by 16 bytes
  static constexpr int LDS_STRIDE = BKB + 16;
  static constexpr int A_BYTES = BM * LDS_STRIDE, B_BYTES = BN * LDS_STRIDE;
  static constexpr int STAGE = A_BYTES + B_BYTES;
  static constexpr int CHUNKS = BKB / 16;
  static constexpr int A_LOADS = (BM * CHUNKS + kThreads - 1) / kThreads;
  static constexpr int B_LOADS = (BN * CHUNKS + kThreads - 1) / kThreads;
  // direct-to-LDS loop: unpadded, XOR-swizzled rows
  static constexpr int DMA_STAGE = (BM + BN) * BKB;
  static constexpr int DMA_STAGES = 4;
  static constexpr int SMEM = PIPE == 2 ? DMA_STAGES * DMA_STAGE : 2 * STAGE;
  static_assert(WM % 32 == 0 && WN % 32 == 0, "tile shape");
};

__device__ __forceinline__ void unpack_i4(const v4i w, v4i &f0, v4i &f1) {
  constexpr int kMask = static_cast<int>(0xF0F0F0F0u);
  f0 = v4i{(w.x << 4) & kMask, w.x & kMask, (w.y << 4) & kMask, w.y & kMask};
  f1 = v4i{(w.z << 4) & kMask, w.z & kMask, (w.w << 4) & kMask, w.w & kMask};
}

template <int N, int I = 0, class F>
__device__ __forceinline__ void static_for(F &&f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<N, I + 1>(f);
  }
}

template <int MODE>
struct FragOps {
  static constexpr int H = MODE == kInt4 ? 2 : 1;  // MFMA k-steps per 32-byte sub-step
  static __device__ __forceinline__ void unpack(const v4i raw, v4i (&u)[H]) {
    if constexpr (MODE == kInt4) {
      unpack_i4(raw, u[0], u[1]);
    } else {
      u[0] = raw;
    }
  }
  // acc += w_frag (rows: output columns n) x x_frag (columns: token rows m)
  template <typename AccT>
  static __device__ __forceinline__ void mma(const v4i x, const v4i w, AccT &acc) {
    if constexpr (MODE == kInt4 || MODE == kInt8) {
      // AccT may be v16f holding integer bit patterns: the fused kernel keeps one accumulator
      // array for both phases so the registers stay in the accumulation file across the switch
      acc = __builtin_bit_cast(AccT, __builtin_amdgcn_mfma_i32_32x32x32_i8(w, x, __builtin_bit_cast(v16i, acc), 0, 0, 0));
    } else if constexpr (MODE == kF16) {
      acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, w), __builtin_bit_cast(v8h, x), acc, 0, 0,
                                                   0);
    } else {
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, w), __builtin_bit_cast(v8bf, x), acc, 0,
                                                    0, 0);
    }
  }
};

// ---------------------------------------------------------------------------------------
// Plain main loop: global -> registers -> padded LDS, double buffered.  Any kbytes % 16 == 0.
template <int ROWS, int LOADS, class C>
struct OperandLoader {
  const uint8_t *ptr[LOADS];
  int lds_off[LOADS];
  int kofs;  // byte offset of this thread's chunk inside a stage
  bool live[LOADS];
  v4i regs[LOADS];

  __device__ __forceinline__ void init(const uint8_t *base, int64_t ld, int rows_valid, int lds_base) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const int item = tid + i * C::kThreads;
      const int row = item / C::CHUNKS, chunk = item % C::CHUNKS;
      live[i] = item < ROWS * C::CHUNKS;
      const int grow = row < rows_valid ? row : rows_valid - 1;  // clamp: rows past the edge are never stored
      ptr[i] = base + int64_t(grow) * ld + chunk * 16;
      lds_off[i] = lds_base + row * C::LDS_STRIDE + chunk * 16;
    }
    kofs = (tid % C::CHUNKS) * 16;
  }
  __device__ __forceinline__ void fetch(int kbyte0, int kbytes) {
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      if (live[i] && kbyte0 + kofs < kbytes) {
        regs[i] = *reinterpret_cast<const v4i *>(ptr[i] + kbyte0);
      } else {
        regs[i] = v4i{0, 0, 0, 0};
      }
    }
  }
  __device__ __forceinline__ void stash(uint8_t *smem, int stage) const {
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      if (live[i]) *reinterpret_cast<v4i *>(smem + stage * C::STAGE + lds_off[i]) = regs[i];
    }
  }
};

template <class C, int MODE, typename AccT>
__device__ __forceinline__ void mainloop_plain(const uint8_t *__restrict__ X, int64_t ldx, int rows_x,
                                               const uint8_t *__restrict__ W, int64_t ldw, int rows_w, int kbytes,
                                               uint8_t *smem, AccT (&acc)[C::MI][C::NI]) {
  using Ops = FragOps<MODE>;
  constexpr int H = Ops::H;
  OperandLoader<C::BM, C::A_LOADS, C> lx;
  OperandLoader<C::BN, C::B_LOADS, C> lw;
  lx.init(X, ldx, rows_x, 0);
  lw.init(W, ldw, rows_w, C::A_BYTES);

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;
  const int x_frag = (wm * C::WM + (lane & 31)) * C::LDS_STRIDE + (lane >> 5) * 16;
  const int w_frag = C::A_BYTES + (wn * C::WN + (lane & 31)) * C::LDS_STRIDE + (lane >> 5) * 16;

  const int stages = (kbytes + C::BKB - 1) / C::BKB;
  lx.fetch(0, kbytes);
  lw.fetch(0, kbytes);
  lx.stash(smem, 0);
  lw.stash(smem, 0);
  __syncthreads();

  for (int kt = 0; kt < stages; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < stages) {
      lx.fetch((kt + 1) * C::BKB, kbytes);
      lw.fetch((kt + 1) * C::BKB, kbytes);
    }
    const uint8_t *sx = smem + cur * C::STAGE + x_frag;
    const uint8_t *sw = smem + cur * C::STAGE + w_frag;
#pragma unroll
    for (int ks = 0; ks < C::BKB / 32; ++ks) {
      v4i ux[C::MI][H];
#pragma unroll
      for (int mi = 0; mi < C::MI; ++mi)
        Ops::unpack(*reinterpret_cast<const v4i *>(sx + mi * 32 * C::LDS_STRIDE + ks * 32), ux[mi]);
#pragma unroll
      for (int ni = 0; ni < C::NI; ++ni) {
        v4i uw[H];
        Ops::unpack(*reinterpret_cast<const v4i *>(sw + ni * 32 * C::LDS_STRIDE + ks * 32), uw);
#pragma unroll
        for (int h = 0; h < H; ++h)
#pragma unroll
          for (int mi = 0; mi < C::MI; ++mi) Ops::mma(ux[mi][h], uw[h], acc[mi][ni]);
      }
    }
    if (kt + 1 < stages) {
      lx.stash(smem, cur ^ 1);
      lw.stash(smem, cur ^ 1);
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------------------------------
// Main loop with direct-to-LDS loads (global_load_lds_dwordx4) over a 4-stage LDS ring.
//
// No register staging: each wave instruction moves 64 x 16 bytes from global memory straight
// into 1 KB of LDS (lane i lands at base + 16 i), i.e. 16 tile rows of 64 bytes.  Rows are
// unpadded; bank conflicts are avoided by an XOR swizzle applied on the global side: lane i of
// a load fetches 16-byte chunk (i % 4) ^ f(row) of its row, and a fragment read of chunk c of
// row r looks at slot c ^ f(r), f(r) = ((r>>1 ^ r>>3) & 1) | ((r>>2 & 1) << 1).  With that f,
// 8 or 16 consecutive rows of one chunk column always fall in distinct 16-byte bank groups
// (measured: zero LDS bank-conflict cycles).
//
// K advances in sub-steps of 32 bytes per row (64 int4 / 32 int8 / 16 half elements), two per
// stage.  While stage k feeds the MFMAs, stage k+1 is complete (its fragments are prefetched
// into registers one or two sub-steps ahead), stage k+2 is landing and stage k+3 is being
// issued.  For int4 the raw nibbles R of sub-step t+2 are read from LDS while sub-step t+1 is
// unpacked into U[1-p] and the MFMAs of sub-step t consume U[p]; sched_group_barrier pins the
// interleave (one MFMA, its share of unpack VALU work, an LDS read every few MFMAs) so the one
// wave per SIMD never waits on an LDS round trip.
// Requires kbytes % 64 == 0: a ragged last stage cannot be zero-filled by the copy engine.

__device__ __forceinline__ int swizzle_f(int r) { return (((r >> 1) ^ (r >> 3)) & 1) | (((r >> 2) & 1) << 1); }


// The pipe streams up to two operand sets back to back through the same LDS ring: set 0 is the
// integer GEMM (qx, qw), set 1 the outlier GEMM (fp_x, fp_w).  Stages are numbered across both,
// so the outlier stages are already landing while the last integer stages are consumed and the
// switch of accumulator type costs no refill of the ring.
template <class C>
struct DmaPipe {
  static constexpr int MI = C::MI, NI = C::NI, NS = C::DMA_STAGES, NF = MI + NI;
  static constexpr int X_REGION = C::BM * 64, STAGE = C::DMA_STAGE;
  static constexpr int X_INSTR = C::BM / 16 / C::WAVES > 0 ? C::BM / 16 / C::WAVES : 1;  // loads per wave and stage
  static constexpr int W_INSTR = C::BN / 16 / C::WAVES > 0 ? C::BN / 16 / C::WAVES : 1;
  static constexpr int kPerStage = X_INSTR + W_INSTR;

  uint8_t *smem;
  uint32_t lds0;
  int wave, x_off, w_off;
  const uint8_t *X[2], *W[2];
  uint32_t vx[2][X_INSTR], vw[2][W_INSTR];
  int stages0, stages;  // stages of set 0, stages of both sets

  // set s: X_s [rows_x, ldx_s bytes], W_s [rows_w, ldw_s bytes], kbytes_s bytes of K (multiple of 64; 0 = absent)
  __device__ __forceinline__ void init(uint8_t *smem_, const uint8_t *X0, int64_t ldx0, const uint8_t *W0,
                                       int64_t ldw0, int kbytes0, const uint8_t *X1, int64_t ldx1,
                                       const uint8_t *W1, int64_t ldw1, int kbytes1, int rows_x, int rows_w) {
    static_assert(C::BM % (16 * C::WAVES) == 0 && C::BN % (16 * C::WAVES) == 0 && NS == 4, "DMA tile shape");
    smem = smem_;
    lds0 = lds_address(smem_);
    const int lane = threadIdx.x & 63;
    wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform: keeps addresses scalar
    const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;
    // global side: lane -> (row within a 16-row block, swizzled chunk); 32-bit offsets from X / W
    const int lrow = lane >> 2;
    const int gchunk = (lane & 3) ^ swizzle_f(lrow);
    X[0] = X0, X[1] = X1, W[0] = W0, W[1] = W1;
    const int64_t ldx[2] = {ldx0, ldx1}, ldw[2] = {ldw0, ldw1};
#pragma unroll
    for (int s = 0; s < 2; ++s) {
#pragma unroll
      for (int j = 0; j < X_INSTR; ++j) {
        const int row = (wave * X_INSTR + j) * 16 + lrow;
        vx[s][j] = static_cast<uint32_t>((row < rows_x ? row : rows_x - 1) * ldx[s] + gchunk * 16);
      }
#pragma unroll
      for (int j = 0; j < W_INSTR; ++j) {
        const int row = (wave * W_INSTR + j) * 16 + lrow;
        vw[s][j] = static_cast<uint32_t>((row < rows_w ? row : rows_w - 1) * ldw[s] + gchunk * 16);
      }
    }
    stages0 = kbytes0 / 64;
    stages = stages0 + kbytes1 / 64;
    // LDS side: fragment j of sub-step ks lives at (operand offset ^ (ks * 32)) + 2048 j
    const int fl = swizzle_f(lane & 15);
    x_off = (wm * C::WM + (lane & 31)) * 64 + (((lane >> 5) ^ fl) << 4);
    w_off = X_REGION + (wn * C::WN + (lane & 31)) * 64 + (((lane >> 5) ^ fl) << 4);
  }

  // Load `idx` (0 .. kPerStage-1) of a stage.  The stage index is clamped: surplus issues re-load the
  // last stage into a dead slot.  Branch-free (selects only) so the loads stay in the main loop's
  // basic block, where they are spread between the MFMAs.
  template <int IDX>
  __device__ __forceinline__ void issue_one(int stage) const {
    const int st = stage < stages ? stage : stages - 1;
    const uint32_t slot = lds0 + (stage & (NS - 1)) * STAGE;
    const bool second = st >= stages0;
    const int kb = (second ? st - stages0 : st) * 64;
    if constexpr (IDX < X_INSTR) {
      dma_load16((second ? X[1] : X[0]) + kb, second ? vx[1][IDX] : vx[0][IDX], slot + (wave * X_INSTR + IDX) * 1024);
    } else {
      constexpr int J = IDX - X_INSTR;
      dma_load16((second ? W[1] : W[0]) + kb, second ? vw[1][J] : vw[0][J],
                 slot + X_REGION + (wave * W_INSTR + J) * 1024);
    }
  }
  template <int FIRST, int COUNT>
  __device__ __forceinline__ void issue_range(int stage) const {
    if constexpr (COUNT > 0) {
      issue_one<FIRST>(stage);
      issue_range<FIRST + 1, COUNT - 1>(stage);
    }
  }
  __device__ __forceinline__ void issue(int stage) const { issue_range<0, kPerStage>(stage); }

  __device__ __forceinline__ const v4i *frag_ptr(int stage, int ks, int j) const {
    const int off = j < MI ? (x_off ^ (ks * 32)) + j * 2048 : (w_off ^ (ks * 32)) + (j - MI) * 2048;
    return reinterpret_cast<const v4i *>(smem + (stage & (NS - 1)) * STAGE + off);
  }

  // Fill the ring: afterwards stages 0 and 1 are visible and stage 2 is in flight.
  __device__ __forceinline__ void start() const {
    issue(0);
    issue(1);
    issue(2);
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(kPerStage));
    __syncthreads();
  }

  // Consume stages [kt_begin, kt_end) in MODE.  On entry stages kt_begin and kt_begin + 1 are
  // visible and kt_begin + 2 is in flight; the same holds for kt_end on exit.
  template <int MODE, typename AccT>
  __device__ __forceinline__ void run(int kt_begin, int kt_end, AccT (&acc)[MI][NI]) const {
    using Ops = FragOps<MODE>;
    constexpr int H = Ops::H;
    // U[p]: operand set consumed by a sub-step of parity p (fragment j < MI: X row block j,
    // fragment MI + j: W column block j).  R (int4 only): raw nibbles, read from LDS two sub-steps
    // ahead of their MFMAs and unpacked one sub-step ahead.
    v4i U[2][NF][H];
    v4i R[NF];
    if constexpr (MODE == kInt4) {
#pragma unroll
      for (int j = 0; j < NF; ++j) R[j] = *frag_ptr(kt_begin, 0, j);
#pragma unroll
      for (int j = 0; j < NF; ++j) Ops::unpack(R[j], U[0][j]);
#pragma unroll
      for (int j = 0; j < NF; ++j) R[j] = *frag_ptr(kt_begin, 1, j);
    } else {
#pragma unroll
      for (int j = 0; j < NF; ++j) U[0][j][0] = *frag_ptr(kt_begin, 0, j);
    }

    // Sub-step of parity P: MFMAs consume U[P]; R (raw, sub-step t+1) is unpacked into U[1-P] and
    // refilled, fragment by fragment, from (rs, rk) (sub-step t+2; for the other modes the fragments
    // of sub-step t+1 go straight into U[1-P]).  `half` selects which half of stage `ld_stage`'s
    // global loads is issued here; in program order one load follows every few fragment reads, which
    // keeps them spread over the MFMAs instead of bunched, where their issue time would stall the
    // matrix pipe.
    auto substep = [&](auto parity, auto half, int rs, int rk, int ld_stage) {
      constexpr int P = decltype(parity)::value;
      constexpr int kLoads = (kPerStage + 1) / 2;
      constexpr int kFirst = decltype(half)::value * kLoads;
      constexpr int kCount = kFirst + kLoads <= kPerStage ? kLoads : kPerStage - kFirst;
      constexpr int kEvery = NF / (kCount > 0 ? kCount : 1) > 0 ? NF / (kCount > 0 ? kCount : 1) : 1;
      auto per_frag = [&](auto jc) {
        constexpr int j = decltype(jc)::value;
        if constexpr (MODE == kInt4) {
          Ops::unpack(R[j], U[1 - P][j]);
          R[j] = *frag_ptr(rs, rk, j);
        } else {
          U[1 - P][j][0] = *frag_ptr(rs, rk, j);
        }
        if constexpr ((j + 1) % kEvery == 0 && (j + 1) / kEvery - 1 < kCount) {
          issue_one<kFirst + (j + 1) / kEvery - 1>(ld_stage);
        }
      };
      static_for<NF>(per_frag);
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int h = 0; h < H; ++h)
#pragma unroll
          for (int mi = 0; mi < MI; ++mi) Ops::mma(U[P][mi][h], U[P][MI + ni][h], acc[mi][ni]);
      constexpr int mfmas = MI * NI * H;
      constexpr int per_read = mfmas / NF > 0 ? mfmas / NF : 1;
#pragma unroll
      for (int i = 0; i < mfmas; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
        if constexpr (MODE == kInt4)
          __builtin_amdgcn_sched_group_barrier(0x002, (12 * NF + mfmas - 1) / mfmas, 0);  // its share of unpack work
        if ((i + 1) % per_read == 0) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
      }
    };

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    for (int kt = kt_begin; kt < kt_end; ++kt) {
      if constexpr (MODE == kInt4) {
        substep(I0{}, I0{}, kt + 1, 0, kt + 3);
        substep(I1{}, I1{}, kt + 1, 1, kt + 3);
      } else {
        substep(I0{}, I0{}, kt, 1, kt + 3);
        substep(I1{}, I1{}, kt + 1, 0, kt + 3);
      }
      // Stage kt+2 has landed (stage kt+3 may stay in flight), then a bare barrier: the LDS reads
      // still outstanding target a slot nobody writes before the next barrier, so they need no wait.
      __builtin_amdgcn_s_waitcnt(vmcnt_imm(kPerStage));
      __builtin_amdgcn_s_barrier();
    }
  }

  // Wait for the surplus loads before LDS is reused or the kernel ends.
  __device__ __forceinline__ void drain() const {
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    __syncthreads();
  }
};

template <class C, int MODE, typename AccT>
__device__ __forceinline__ void mainloop_dma(const uint8_t *__restrict__ X, int64_t ldx, int rows_x,
                                             const uint8_t *__restrict__ W, int64_t ldw, int rows_w, int kbytes,
                                             uint8_t *smem, AccT (&acc)[C::MI][C::NI]) {
  DmaPipe<C> pipe;
  pipe.init(smem, X, ldx, W, ldw, kbytes, X, ldx, W, ldw, 0, rows_x, rows_w);
  pipe.start();
  pipe.template run<MODE>(0, pipe.stages, acc);
  pipe.drain();
}

template <class C, int MODE, typename AccT>
__device__ __forceinline__ void run_mainloop(const uint8_t *__restrict__ X, int64_t ldx, int rows_x,
                                             const uint8_t *__restrict__ W, int64_t ldw, int rows_w, int kbytes,
                                             uint8_t *smem, AccT (&acc)[C::MI][C::NI]) {
  if constexpr (C::PIPE == 2) {
    mainloop_dma<C, MODE>(X, ldx, rows_x, W, ldw, rows_w, kbytes, smem, acc);
  } else {
    mainloop_plain<C, MODE>(X, ldx, rows_x, W, ldw, rows_w, kbytes, smem, acc);
  }
}

// Workgroup id -> tile.  Hardware deals consecutive workgroup ids round-robin to the 8 XCDs;
// ids congruent mod 8 therefore share an L2.  Give each XCD a contiguous run of tiles, with M
// fastest, so concurrently resident tiles of an XCD share W rows and cover all of X.
// `bid` is the workgroup's index inside its launch region; regions start at multiples of 8.
__device__ __forceinline__ bool tile_of_block(int bid, int tiles_m, int tiles_n, int &tm, int &tn) {
  const int total = tiles_m * tiles_n;
  const int per_xcd = (total + 7) / 8;
  const int logical = (bid % 8) * per_xcd + bid / 8;
  if (logical >= total) return false;
  tm = logical % tiles_m;
  tn = logical / tiles_m;
  return true;
}

// Accumulator register v of a 32x32 block, for this lane: token row m = lane % 32, output
// column n = 8 * (v / 4) + 4 * (lane / 32) + v % 4: four consecutive columns per group of four.
__device__ __forceinline__ int acc_col(int g, int lane) { return 8 * g + 4 * (lane >> 5); }

// Writes one 32-row x WN-column block of results (one `mi` block of a wave) to global memory
// through a wave-private LDS staging area, so that every store instruction writes whole
// contiguous row segments (>= 128 bytes per row) instead of 8/16-byte pieces of 32 rows:
// partial-sector writes cost the memory system several times the bytes they carry.
// Staging rows are padded by 16 bytes, which keeps both the 8/16-byte writes of the MFMA
// layout and the 16-byte row-wise reads free of bank conflicts.
template <class C, typename T>
struct BlockStore {
  static constexpr int kRowBytes = C::WN * int(sizeof(T)) + 16;
  static constexpr int kBytes = 32 * kRowBytes;          // per wave
  static constexpr int kLanesPerRow = C::WN * int(sizeof(T)) / 16;
  static constexpr int kRowsPerInstr = 64 / kLanesPerRow;
  static constexpr int kElems = 16 / int(sizeof(T));      // elements per 16-byte piece

  // four consecutive columns (ni, g) of this lane's row
  static __device__ __forceinline__ void put(uint8_t *stage, int lane, int ni, int g, const T (&v)[4]) {
    uint8_t *dst = stage + (lane & 31) * kRowBytes + (ni * 32 + acc_col(g, lane)) * int(sizeof(T));
    if constexpr (sizeof(T) == 4) {
      *reinterpret_cast<v4i *>(dst) = v4i{int(v[0]), int(v[1]), int(v[2]), int(v[3])};
    } else {
      *reinterpret_cast<uint2 *>(dst) =
          make_uint2(uint32_t(v[0]) | (uint32_t(v[1]) << 16), uint32_t(v[2]) | (uint32_t(v[3]) << 16));
    }
  }

  // the same for 16-bit elements that are already packed in pairs
  static __device__ __forceinline__ void put_pairs(uint8_t *stage, int lane, int ni, int g, uint32_t lo, uint32_t hi) {
    static_assert(sizeof(T) == 2, "16-bit elements");
    *reinterpret_cast<uint2 *>(stage + (lane & 31) * kRowBytes + (ni * 32 + acc_col(g, lane)) * 2) = make_uint2(lo, hi);
  }

  // the reverse direction: g[row * ld + col] (rows < rows_valid, cols < cols_valid, zeros elsewhere) -> staged block,
  // as 16-byte pieces of row segments; get() then reads this lane's four consecutive columns (ni, g) of its row
  static __device__ __forceinline__ void load(uint8_t *stage, int lane, const T *g, int64_t ld, int rows_valid,
                                              int cols_valid, bool vec) {
    __builtin_amdgcn_wave_barrier();  // earlier reads of the staging block by other lanes are done (same wave: in order)
#pragma unroll
    for (int it = 0; it < 32 / kRowsPerInstr; ++it) {
      const int r = it * kRowsPerInstr + lane / kLanesPerRow;
      const int c = (lane % kLanesPerRow) * kElems;
      v4i piece = v4i{0, 0, 0, 0};
      if (r < rows_valid) {
        const T *src = g + int64_t(r) * ld + c;
        if (vec && c + kElems <= cols_valid) {
          piece = *reinterpret_cast<const v4i *>(src);
        } else {
          T tmp[kElems] = {};
#pragma unroll
          for (int e = 0; e < kElems; ++e)
            if (c + e < cols_valid) tmp[e] = src[e];
          __builtin_memcpy(&piece, tmp, 16);
        }
      }
      *reinterpret_cast<v4i *>(stage + r * kRowBytes + (lane % kLanesPerRow) * 16) = piece;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  static __device__ __forceinline__ void get(const uint8_t *stage, int lane, int ni, int g, T (&v)[4]) {
    static_assert(sizeof(T) == 2, "16-bit elements");
    const uint2 w = *reinterpret_cast<const uint2 *>(stage + (lane & 31) * kRowBytes + (ni * 32 + acc_col(g, lane)) * 2);
    v[0] = static_cast<T>(w.x & 0xFFFFu), v[1] = static_cast<T>(w.x >> 16);
    v[2] = static_cast<T>(w.y & 0xFFFFu), v[3] = static_cast<T>(w.y >> 16);
  }

  // interior block: the 32 / kRowsPerInstr pieces of a staged block, and their places in global memory
  static constexpr int kIters = 32 / kRowsPerInstr;
  static __device__ __forceinline__ void read_block(const uint8_t *stage, int lane, v4i (&piece)[kIters]) {
#pragma unroll
    for (int it = 0; it < kIters; ++it)
      piece[it] = *reinterpret_cast<const v4i *>(stage + (it * kRowsPerInstr + lane / kLanesPerRow) * kRowBytes +
                                                 (lane % kLanesPerRow) * 16);
  }
  static __device__ __forceinline__ void write_block(const v4i (&piece)[kIters], int lane, T *g, int64_t ld) {
#pragma unroll
    for (int it = 0; it < kIters; ++it)
      store_piece(piece[it], g + int64_t(it * kRowsPerInstr + lane / kLanesPerRow) * ld + (lane % kLanesPerRow) * kElems);
  }
  // One 16-byte piece of an output row.  The fp16 / bf16 layer output is written once and not read again by this
  // launch: a streaming (non-temporal) store keeps its 100+ MB from displacing the operand lines that the tiles of
  // an XCD share through L2 (70B gate_proj, 2048 tokens: GEMM 0.274 -> 0.242 ms).  The int32 product of the
  // stand-alone GEMMs is read back at once by a dequantize kernel and keeps the default policy.
  static __device__ __forceinline__ void store_piece(const v4i &piece, T *dst) {
    if constexpr (sizeof(T) == 2) {
      __builtin_nontemporal_store(piece, reinterpret_cast<v4i *>(dst));
    } else {
      *reinterpret_cast<v4i *>(dst) = piece;
    }
  }

  // staged block -> g[row * ld + col], rows < rows_valid, cols < cols_valid
  static __device__ __forceinline__ void flush(const uint8_t *stage, int lane, T *g, int64_t ld, int rows_valid,
                                               int cols_valid, bool vec) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (vec && rows_valid >= 32 && cols_valid >= C::WN) {  // interior block (wave-uniform): straight-line code
      constexpr int kIters = 32 / kRowsPerInstr;
      v4i piece[kIters];
#pragma unroll
      for (int it = 0; it < kIters; ++it)
        piece[it] = *reinterpret_cast<const v4i *>(stage + (it * kRowsPerInstr + lane / kLanesPerRow) * kRowBytes +
                                                   (lane % kLanesPerRow) * 16);
#pragma unroll
      for (int it = 0; it < kIters; ++it)
        store_piece(piece[it], g + int64_t(it * kRowsPerInstr + lane / kLanesPerRow) * ld + (lane % kLanesPerRow) * kElems);
      __builtin_amdgcn_wave_barrier();
      return;
    }
#pragma unroll
    for (int it = 0; it < 32 / kRowsPerInstr; ++it) {
      const int r = it * kRowsPerInstr + lane / kLanesPerRow;
      const int c = (lane % kLanesPerRow) * kElems;
      const v4i piece = *reinterpret_cast<const v4i *>(stage + r * kRowBytes + (lane % kLanesPerRow) * 16);
      if (r >= rows_valid) continue;
      T *dst = g + int64_t(r) * ld + c;
      if (vec && c + kElems <= cols_valid) {
        store_piece(piece, dst);
      } else {
        T tmp[kElems];
        __builtin_memcpy(tmp, &piece, 16);
#pragma unroll
        for (int e = 0; e < kElems; ++e)
          if (c + e < cols_valid) dst[e] = tmp[e];
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
};

// C [M, ldc] int32; this launch covers N columns starting at C's column 0 (host offsets pointers).
struct I32Args {
  const uint8_t *X, *W;
  int32_t *C;
  int M, N, ldc, kbytes;
};

template <class C, int MODE>
__device__ __forceinline__ void i32_tile(const I32Args &a, int tm, int tn, uint8_t *smem) {
  const uint8_t *__restrict__ X = a.X;
  const uint8_t *__restrict__ W = a.W;
  int32_t *__restrict__ Cm = a.C;
  const int M = a.M, N = a.N, ldc = a.ldc, kbytes = a.kbytes;
  const int m0 = tm * C::BM, n0 = tn * C::BN;
  v16i acc[C::MI][C::NI];
#pragma unroll
  for (int mi = 0; mi < C::MI; ++mi)
#pragma unroll
    for (int ni = 0; ni < C::NI; ++ni)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0;
  run_mainloop<C, MODE>(X + int64_t(m0) * kbytes, kbytes, M - m0, W + int64_t(n0) * kbytes, kbytes, N - n0, kbytes,
                        smem, acc);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;
  constexpr int kShift = MODE == kInt4 ? 8 : 0;
  using Store = BlockStore<C, int32_t>;
  static_assert(Store::kBytes * C::WAVES <= C::SMEM, "staging fits in the (now idle) operand buffers");
  uint8_t *stage = smem + wave * Store::kBytes;
  const bool vec = (ldc & 3) == 0 && (reinterpret_cast<uintptr_t>(Cm) & 15) == 0;
  const int nw = n0 + wn * C::WN;
#pragma unroll
  for (int mi = 0; mi < C::MI; ++mi) {
    const int mb = m0 + wm * C::WM + mi * 32;
#pragma unroll
    for (int ni = 0; ni < C::NI; ++ni)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int32_t v[4] = {acc[mi][ni][4 * g] >> kShift, acc[mi][ni][4 * g + 1] >> kShift,
                              acc[mi][ni][4 * g + 2] >> kShift, acc[mi][ni][4 * g + 3] >> kShift};
        Store::put(stage, lane, ni, g, v);
      }
    if (mb < M && nw < N)
      Store::flush(stage, lane, Cm + int64_t(mb) * ldc + nw, ldc, M - mb, N - nw, vec);
  }
}

template <class C, int MODE>
__global__ __launch_bounds__(C::kThreads) void gemm_i32_kernel(I32Args a, int tiles_m, int tiles_n) {
  extern __shared__ __align__(16) uint8_t smem[];
  int tm, tn;
  if (!tile_of_block(blockIdx.x, tiles_m, tiles_n, tm, tn)) return;
  i32_tile<C, MODE>(a, tm, tn, smem);
}

// ---- the reference's fused GEMM + dequantize ops: exact integer product, fp16-arithmetic epilogue -----------------
// (reference: src/asymmetric/fused_dequantize.cu:9-119 with include/asymmetric/epilogue/thread/
// linear_combination_dequant.h:155-162, and src/symmetric/fused_dequantize.cu:9-107 with
// include/symmetric/epilogue/thread/linear_combination_dequant.h:149-150).  Every operation rounds to fp16:
//   asymmetric: ((h(acc) * s_col) * s_row + (zero_row + h(shift) * s_row) * w_red) + y
//   symmetric:  ((h(acc) * s_row) * s_col) + y
// h(acc): int32 -> fp16, round to nearest even, +-inf above 65519.  One launch: the epilogue runs on the accumulators
// of the tile (no int32 matrix in memory), y is read and the result written as 16-byte pieces of row segments.
struct ChainArgs {
  const uint16_t *s_row, *s_col, *zero_row, *w_red, *y;  // zero_row, w_red: NULL for the symmetric form
  uint16_t *out;
  int ldy;          // row stride of y and out in elements
  uint16_t shift;   // fp16 bit pattern of the shift value (asymmetric)
};

template <class C, int MODE, bool ASYM>
__device__ __forceinline__ void chain_tile(const I32Args &a, const ChainArgs &e, int tm, int tn, uint8_t *smem) {
  const int M = a.M, N = a.N, kbytes = a.kbytes;
  const int m0 = tm * C::BM, n0 = tn * C::BN;
  v16i acc[C::MI][C::NI];
#pragma unroll
  for (int mi = 0; mi < C::MI; ++mi)
#pragma unroll
    for (int ni = 0; ni < C::NI; ++ni)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0;
  run_mainloop<C, MODE>(a.X + int64_t(m0) * kbytes, kbytes, M - m0, a.W + int64_t(n0) * kbytes, kbytes, N - n0, kbytes,
                        smem, acc);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;
  constexpr int kShift = MODE == kInt4 ? 8 : 0;
  using Store = BlockStore<C, uint16_t>;
  static_assert(Store::kBytes * C::WAVES <= C::SMEM, "staging fits in the (now idle) operand buffers");
  uint8_t *stage = smem + wave * Store::kBytes;
  const bool vec = (e.ldy & 7) == 0 && (reinterpret_cast<uintptr_t>(e.out) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(e.y) & 15) == 0;
  const int nw = n0 + wn * C::WN;
  auto h = [](uint16_t b) { return __builtin_bit_cast(_Float16, b); };
  const _Float16 shift = h(e.shift);
#pragma unroll
  for (int mi = 0; mi < C::MI; ++mi) {
    const int mb = m0 + wm * C::WM + mi * 32;
    if (!(mb < M && nw < N)) continue;  // wave-uniform
    // y of this 32-row block through the staging area: global -> LDS as row segments, LDS -> this lane's places
    Store::load(stage, lane, e.y + int64_t(mb) * e.ldy + nw, e.ldy, M - mb, N - nw, vec);
    const int r = mb + (lane & 31) < M ? mb + (lane & 31) : M - 1;
    const _Float16 sr = h(e.s_row[r]);
    _Float16 u0 = static_cast<_Float16>(0);
    if constexpr (ASYM) u0 = h(e.zero_row[r]) + shift * sr;  // (zero_row + h(shift) * s_row), two roundings
#pragma unroll
    for (int ni = 0; ni < C::NI; ++ni)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int c0 = nw + ni * 32 + acc_col(g, lane);
        uint16_t yv[4], o[4];
        Store::get(stage, lane, ni, g, yv);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int c = c0 + k < N ? c0 + k : N - 1;
          _Float16 t = static_cast<_Float16>(static_cast<float>(acc[mi][ni][4 * g + k] >> kShift));
          if constexpr (ASYM) {
            t = t * h(e.s_col[c]);
            t = t * sr;
            t = t + u0 * h(e.w_red[c]);
          } else {
            t = t * sr;
            t = t * h(e.s_col[c]);
          }
          t = t + h(yv[k]);
          o[k] = __builtin_bit_cast(uint16_t, t);
        }
        Store::put(stage, lane, ni, g, o);
      }
    Store::flush(stage, lane, e.out + int64_t(mb) * e.ldy + nw, e.ldy, M - mb, N - nw, vec);
  }
}

template <class C, int MODE, bool ASYM>
__global__ __launch_bounds__(C::kThreads) void gemm_chain_kernel(I32Args a, ChainArgs e, int tiles_m, int tiles_n) {
  extern __shared__ __align__(16) uint8_t smem[];
  int tm, tn;
  if (!tile_of_block(blockIdx.x, tiles_m, tiles_n, tm, tn)) return;
  chain_tile<C, MODE, ASYM>(a, e, tm, tn, smem);
}

// One launch, two tile shapes.  Workgroup ids [lead, lead + wide_blocks) take CW tiles of `wide`,
// the ids before and after take CT tiles of `tail`.  Hardware starts workgroups in id order as CUs
// free up, so the narrow tiles at the end even out the schedule; the `lead` narrow tiles at the
// front put part of the CUs half a tile ahead of the others, so that the tiles' store bursts do
// not all hit memory at the same moment.  lead and wide_blocks are multiples of 8.
struct SplitGrid {
  int tiles_m, tiles_n_wide, tiles_n_tail, lead, wide_blocks;
  // returns 0: no tile, 1: wide tile, 2: tail tile
  __device__ __forceinline__ int locate(int bid, int &tm, int &tn) const {
    if (bid >= lead && bid < lead + wide_blocks) return tile_of_block(bid - lead, tiles_m, tiles_n_wide, tm, tn) ? 1 : 0;
    const int local = bid < lead ? bid : bid - wide_blocks;
    return tile_of_block(local, tiles_m, tiles_n_tail, tm, tn) ? 2 : 0;
  }
};

template <class CW, class CT, int MODE>
__global__ __launch_bounds__(CW::kThreads) void gemm_i32_split_kernel(I32Args wide, I32Args tail, SplitGrid grid) {
  static_assert(CW::kThreads == CT::kThreads, "one block size");
  extern __shared__ __align__(16) uint8_t smem[];
  int tm, tn;
  const int kind = grid.locate(blockIdx.x, tm, tn);
  if (kind == 1) {
    i32_tile<CW, MODE>(wide, tm, tn, smem);
  } else if (kind == 2) {
    i32_tile<CT, MODE>(tail, tm, tn, smem);
  }
}


struct FusedArgs {
  const uint8_t *qx, *qw;
  const uint16_t *meta, *s_col, *w_red, *fp_x, *fp_w, *bias;
  uint16_t *out;
  int M, N, ldo, kbytes, F;  // N: columns of this launch; ldo: row stride of out in elements
  int meta_stride;           // 2: (scale, zero) pairs; 1: scales only (symmetric)
  float shift;
};

// Explicit moves between the accumulation registers (where the MFMA results live) and the vector
// registers (the only ones VALU instructions can touch).  Spelled out so that the conversion
// between the two MFMA phases streams through a handful of vector registers; left to itself the
// register allocator copies all 256 accumulators out at once and spills.
// (Hazards: a read that follows an MFMA writing the same accumulator needs that MFMA's passes to have finished;
// the callers put 2 x s_nop 15 between the last MFMA and the first read, more than the 18 wait states the
// longest MFMA used here asks for.  Between VALU instructions and these moves the hardware interlocks, as for any
// VALU pair; the compiler schedules its own MFMAs after an agpr_write through the register dependence.)
__device__ __forceinline__ float agpr_read(float a) {
  float v;
  asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(a));
  return v;
}
__device__ __forceinline__ float agpr_write(float v) {
  float a;
  asm volatile("v_accvgpr_write_b32 %0, %1" : "=a"(a) : "v"(v));
  return a;
}

// Per-tile row and column vectors, widened to fp32 once and kept in LDS behind the operand ring:
//   s_col[BN], w_red[BN], bias[BN], s_row[BM], zs[BM] with zs = zero + 2^(bits-1) * s_row.
template <class C>
struct TileVectors {
  static constexpr int kBytes = (3 * C::BN + 2 * C::BM) * 4;
  float *scol, *wred, *bias, *srow, *zs;
  __device__ __forceinline__ explicit TileVectors(uint8_t *base) {
    scol = reinterpret_cast<float *>(base);
    wred = scol + C::BN;
    bias = wred + C::BN;
    srow = bias + C::BN;
    zs = srow + C::BM;
  }
  template <bool BF16>
  __device__ __forceinline__ void fill(const FusedArgs &p, int m0, int n0) const {
    for (int i = threadIdx.x; i < C::BN; i += C::kThreads) {
      const int n = n0 + i < p.N ? n0 + i : p.N - 1;
      scol[i] = to_f32<BF16>(p.s_col[n]);
      wred[i] = p.w_red ? to_f32<BF16>(p.w_red[n]) : 0.0f;
      bias[i] = p.bias ? to_f32<BF16>(p.bias[n]) : 0.0f;
    }
    for (int i = threadIdx.x; i < C::BM; i += C::kThreads) {
      const int64_t m = m0 + i < p.M ? m0 + i : p.M - 1;
      const float s = to_f32<BF16>(p.meta[m * p.meta_stride]);
      srow[i] = s;
      zs[i] = p.w_red ? to_f32<BF16>(p.meta[2 * m + 1]) + p.shift * s : 0.0f;
    }
  }
};

template <class C>
constexpr int fused_smem() {
  return C::SMEM + TileVectors<C>::kBytes;
}

template <class C, int MODE, bool BF16>
__device__ __forceinline__ void fused_tile(const FusedArgs &p, int tm, int tn, uint8_t *smem) {
  const int m0 = tm * C::BM, n0 = tn * C::BN;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;
  const TileVectors<C> tv(smem + C::SMEM);
  tv.template fill<BF16>(p, m0, n0);  // made visible by the first barrier of the main loop

  v16f accf[C::MI][C::NI];  // integer bit patterns during the first phase, floats afterwards
  {
    v16f (&acc)[C::MI][C::NI] = accf;
#pragma unroll
    for (int mi = 0; mi < C::MI; ++mi)
#pragma unroll
      for (int ni = 0; ni < C::NI; ++ni)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0.0f;
    const uint8_t *qx = p.qx + int64_t(m0) * p.kbytes, *qw = p.qw + int64_t(n0) * p.kbytes;
    const uint8_t *fx = reinterpret_cast<const uint8_t *>(p.fp_x) + int64_t(m0) * p.F * 2;
    const uint8_t *fw = reinterpret_cast<const uint8_t *>(p.fp_w) + int64_t(n0) * p.F * 2;
    DmaPipe<C> pipe;
    if constexpr (C::PIPE == 2) {
      pipe.init(smem, qx, p.kbytes, qw, p.kbytes, p.kbytes, fx, int64_t(p.F) * 2, fw, int64_t(p.F) * 2, p.F * 2,
                p.M - m0, p.N - n0);
      pipe.start();
      pipe.template run<MODE>(0, pipe.stages0, acc);
    } else {
      mainloop_plain<C, MODE>(qx, p.kbytes, p.M - m0, qw, p.kbytes, p.N - n0, p.kbytes, smem, acc);
    }
    // acc -> f32(acc) * (s_row * s_col) + (zs * w_red + bias), in place.  The int4 accumulators carry a factor 256;
    // it is removed by scaling s_row with 2^-8 instead of shifting: both are exact, so
    // f32(256 a) * ((s_row 2^-8) s_col) rounds to the same float as f32(a) * (s_row s_col).  The zero-point and
    // bias term is the addend of the multiply: the epilogue only converts and stores.
    float srow[C::MI], zsr[C::MI];
#pragma unroll
    for (int mi = 0; mi < C::MI; ++mi) {
      srow[mi] = tv.srow[wm * C::WM + mi * 32 + (lane & 31)] * (MODE == kInt4 ? 0.00390625f : 1.0f);
      zsr[mi] = tv.zs[wm * C::WM + mi * 32 + (lane & 31)];
    }
    // one 32x32 block (a 16-register accumulator tuple) at a time
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
          const float raw = agpr_read(acc[mi][ni][v]);
          accf[mi][ni][v] = agpr_write(__builtin_fmaf(static_cast<float>(__float_as_int(raw)), srow[mi] * scv[v],
                                                      __builtin_fmaf(zsr[mi], wrv[v], bsv[v])));
        }
      }
    }
    if constexpr (C::PIPE == 2) {
      pipe.template run<BF16 ? kBF16 : kF16>(pipe.stages0, pipe.stages, accf);
      pipe.drain();
    }
  }
  if constexpr (C::PIPE != 2) {
    if (p.F > 0) {
      mainloop_plain<C, BF16 ? kBF16 : kF16>(reinterpret_cast<const uint8_t *>(p.fp_x) + int64_t(m0) * p.F * 2,
                                             int64_t(p.F) * 2, p.M - m0,
                                             reinterpret_cast<const uint8_t *>(p.fp_w) + int64_t(n0) * p.F * 2,
                                             int64_t(p.F) * 2, p.N - n0, p.F * 2, smem, accf);
    }
  }
  // out = storage(accf), written through the staging area
  using Store = BlockStore<C, uint16_t>;
  static_assert(Store::kBytes * C::WAVES <= C::SMEM, "staging fits in the (now idle) operand buffers");
  uint8_t *stage = smem + wave * Store::kBytes;
  const bool vec = (p.ldo & 7) == 0 && (reinterpret_cast<uintptr_t>(p.out) & 15) == 0;
  const int nw = n0 + wn * C::WN;
#pragma unroll
  for (int mi = 0; mi < C::MI; ++mi) {
    const int mb = m0 + wm * C::WM + mi * 32;
#pragma unroll
    for (int ni = 0; ni < C::NI; ++ni)
#pragma unroll
      for (int g = 0; g < 4; ++g)
        Store::put_pairs(stage, lane, ni, g, pack2_from_f32<BF16>(accf[mi][ni][4 * g], accf[mi][ni][4 * g + 1]),
                         pack2_from_f32<BF16>(accf[mi][ni][4 * g + 2], accf[mi][ni][4 * g + 3]));
    if (mb < p.M && nw < p.N) Store::flush(stage, lane, p.out + int64_t(mb) * p.ldo + nw, p.ldo, p.M - mb, p.N - nw, vec);
    __builtin_amdgcn_sched_barrier(0);
  }
}

template <class C, int MODE, bool BF16>
__global__ __launch_bounds__(C::kThreads) void gemm_fused_kernel(FusedArgs p, int tiles_m, int tiles_n) {
  extern __shared__ __align__(16) uint8_t smem[];
  int tm, tn;
  if (!tile_of_block(blockIdx.x, tiles_m, tiles_n, tm, tn)) return;
  fused_tile<C, MODE, BF16>(p, tm, tn, smem);
}

// One launch, two tile shapes (see gemm_i32_split_kernel).
template <class CW, class CT, int MODE, bool BF16>
__global__ __launch_bounds__(CW::kThreads) void gemm_fused_split_kernel(FusedArgs wide, FusedArgs tail,
                                                                        SplitGrid grid) {
  static_assert(CW::kThreads == CT::kThreads, "one block size");
  extern __shared__ __align__(16) uint8_t smem[];
  int tm, tn;
  const int kind = grid.locate(blockIdx.x, tm, tn);
  if (kind == 1) {
    fused_tile<CW, MODE, BF16>(wide, tm, tn, smem);
  } else if (kind == 2) {
    fused_tile<CT, MODE, BF16>(tail, tm, tn, smem);
  }
}

}  // namespace quik
