// int8 x int8 fused GEMM (W8A8 MixedQLinear forward) on operand buffers stored in tile order.
//
// Same idea as the 6-bit path (gemm_fp6.h), with v_mfma_i32_32x32x32_i8: both operands are stored as the
// sequence of LDS images the tiles need, so that a copy instruction (global_load_lds_dwordx4, 64 lanes x
// 16 bytes) moves one contiguous, aligned kilobyte and every cache line is requested once per tile.  With
// row-major int8 operands a tile asks for 64 bytes per row and stage, i.e. for every line twice, two stages
// apart, and the 64 KB it touches meanwhile do not survive in the 32 KB vector cache: the W8A8 loop needs
// 64 bytes per cycle from L2 then, which is all the path delivers.
//
// Operand format (tile8_layout in fp6_format.h): rows in blocks of 64; unit (block B, step s) is 2 KB:
//   [0, 1024) rows 0..31 of the block, [1024, 2048) rows 32..63; row r at 32 r; 16-byte chunk h (K elements
//   16 h .. 16 h + 15 of the step's 32) in slot h ^ ((r >> 3) & 1).
// A block's units are contiguous: K / 32 integer steps, then F / 16 outlier steps (16 fp16 / bf16 values =
// 32 bytes per row, same image).  Needs K % 64 == 0 and F % 32 == 0 (steps are consumed in pairs).
//
// Pipeline: ring of 6 LDS slots of one step each ((BM + BN) x 32 bytes), mirroring the units; while step j
// feeds the MFMAs, the fragments of step j + 1 are read into the second register set and steps j + 2 .. j + 5
// are landing; copies go one by one between groups of MFMAs (see gemm_fp6.h for the reasons).
#pragma once
#include "gemm_fp6.h"

namespace quik {

template <class C>
struct Tile8Pipe {
  static constexpr int MI = C::MI, NI = C::NI, NS = 6, NF = MI + NI, MM = MI * NI;
  static_assert(C::WM % 64 == 0 && C::WN % 64 == 0, "a wave's rows start at a 64-row block");
  static_assert(C::WAVES == 4 || C::WAVES == 8, "copy assignment below");
  static constexpr int W_OFF = C::BM * 32;
  static constexpr int STAGE = (C::BM + C::BN) * 32;
  static constexpr int SMEM = NS * STAGE;
  // Copies per step: 2 per 64-row block.  Every wave copies one whole block from its source A (X block w, or W
  // block w - XB), and NB further kilobytes from its source B:
  //   four waves, 256x256: W block w (2);  256x128: W block w % 2, piece w / 2 (1);  128x128: none;
  //   eight waves, 256x256: none.
  static constexpr int XB = C::BM / 64, WB = C::BN / 64;
  static constexpr int NB = C::WAVES == 8 ? 0 : XB + WB == 8 ? 2 : XB + WB == 6 ? 1 : 0;
  static_assert((XB == 4 && (WB == 4 || WB == 2)) || (XB == 2 && WB == 2), "supported tile shapes");
  static_assert(C::WAVES == 4 || XB + WB == 8, "eight waves copy eight blocks");
  static constexpr int P = 2 + NB;  // copies per wave and step
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
  uint32_t x_head, w_head;  // this lane's fragment offsets inside a slot (fragment j: + 2048 (j / 2) + 1024 (j % 2))
  uint32_t x_head3[3], w_head3[3];  // the same inside slots 0, 2, 4

  // unit0: first unit (step) of every block to copy; n_int / n_f: integer and outlier steps from there on
  // (-1: all of the block's, from its first unit)
  __device__ __forceinline__ void init(uint8_t *smem_, const uint8_t *xbuf, const Tile8Layout &lx, int64_t xb0,
                                       const uint8_t *wbuf, const Tile8Layout &lw, int64_t wb0, int unit0 = 0,
                                       int n_int = -1, int n_f = -1) {
    smem = smem_;
    lds0 = lds_address(smem_);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;
    auto block_ptr = [&](bool is_x, int blk) {
      const Tile8Layout &l = is_x ? lx : lw;
      int64_t B = (is_x ? xb0 : wb0) + blk;
      B = B < l.blocks ? B : l.blocks - 1;  // blocks past the matrix: any valid block, results never stored
      return (is_x ? xbuf : wbuf) + B * l.block_bytes + int64_t(unit0) * 2048;
    };
    {
      const bool is_x = wave < XB;
      const int blk = is_x ? wave : wave - XB;
      pa = block_ptr(is_x, blk);
      da = (is_x ? 0 : W_OFF) + blk * 2048;
    }
    pb = pa;
    db = da;
    if constexpr (NB == 2) {
      pb = block_ptr(false, wave);
      db = W_OFF + wave * 2048;
    } else if constexpr (NB == 1) {
      pb = block_ptr(false, wave & 1) + (wave >> 1) * 1024;
      db = W_OFF + (wave & 1) * 2048 + (wave >> 1) * 1024;
    }
    lane16 = lane * 16;
    fill = lds0;
    rd = 0;
    steps0 = n_int < 0 ? static_cast<int>(lx.steps) : n_int;
    steps = steps0 + (n_f < 0 ? static_cast<int>(lx.fsteps) : n_f);
    left = steps;
    const int r = lane & 31, h = lane >> 5;
    const int slot16 = (h ^ ((r >> 3) & 1)) << 4;
    x_head = (wm * C::WM / 64) * 2048 + r * 32 + slot16;
    w_head = W_OFF + (wn * C::WN / 64) * 2048 + r * 32 + slot16;
#pragma unroll
    for (int q = 0; q < 3; ++q) {
      x_head3[q] = x_head + q * 2 * STAGE;
      w_head3[q] = w_head + q * 2 * STAGE;
    }
  }

  // Copy G of the step being copied (FS: slot when known at compile time, else `fill`); after the last one the
  // scalar bookkeeping.  Past the last step the pointers stop and the last step is copied again into a slot
  // nobody reads.
  template <int G, int FS = -1>
  __device__ __forceinline__ void issue_one() {
    const uint32_t slot = FS < 0 ? fill : lds0 + (FS < 0 ? 0 : FS) * STAGE;
    if constexpr (G < 2) {
      dma_load16k<G * 1024>(pa, lane16, slot + da);
    } else {
      dma_load16k<(G - 2) * 1024>(pb, lane16, slot + db);
    }
    if constexpr (G == P - 1) {
      const int adv = left > 1 ? 2048 : 0;
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

  // Fill the ring: afterwards steps 0 and 1 are visible and steps 2 .. 4 are in flight.
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

  template <int J, int RS = -1>
  __device__ __forceinline__ void read_one(v4i (&f)[NF]) const {
    constexpr int jj = J < MI ? J : J - MI;
    if constexpr (RS < 0) {
      f[J] = *reinterpret_cast<const v4i *>(smem + rd + (J < MI ? x_head : w_head) + (jj >> 1) * 2048 + (jj & 1) * 1024);
    } else {
      constexpr int q = (RS < 0 ? 0 : RS) / 2, odd = ((RS < 0 ? 0 : RS) % 2) * STAGE;
      f[J] = *reinterpret_cast<const v4i *>(smem + (J < MI ? x_head3[q] : w_head3[q]) + odd + (jj >> 1) * 2048 +
                                            (jj & 1) * 1024);
    }
  }
  template <int J = 0>
  __device__ __forceinline__ void read_all(v4i (&f)[NF]) {
    if constexpr (J < NF) {
      read_one<J>(f);
      read_all<J + 1>(f);
    } else {
      next_read_slot();
    }
  }
  template <int RS, int LO, int HI>
  __device__ __forceinline__ void chunk_reads(v4i (&nf)[NF]) const {
    if constexpr (LO < HI) {
      read_one<LO, RS>(nf);
      chunk_reads<RS, LO + 1, HI>(nf);
    }
  }
  template <int MODE, int LO, int HI>
  static __device__ __forceinline__ void chunk_mfmas(const v4i (&cf)[NF], v16f (&acc)[MI][NI]) {
    if constexpr (LO < HI) {
      FragOps<MODE>::mma(cf[LO % MI], cf[MI + LO / MI], acc[LO % MI][LO / MI]);
      chunk_mfmas<MODE, LO + 1, HI>(cf, acc);
    }
  }

  // One step in P chunks: a share of the MFMAs (fragments in `cf`), of the next step's fragment reads (into
  // `nf`) and one copy of the step five ahead; then wait until the step after next has landed and a barrier.
  template <int MODE, int RS = -1, int FS = -1, int G = 0>
  __device__ __forceinline__ void step(const v4i (&cf)[NF], v4i (&nf)[NF], v16f (&acc)[MI][NI]) {
    if constexpr (G < P) {
      constexpr int r_lo = G * NF / P, r_hi = (G + 1) * NF / P, m_lo = G * MM / P, m_hi = (G + 1) * MM / P;
      chunk_reads<RS, r_lo, r_hi>(nf);
      chunk_mfmas<MODE, m_lo, m_hi>(cf, acc);
#pragma unroll
      for (int i = m_lo; i < m_hi; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, ((r_hi - r_lo) + (m_hi - m_lo) - 1) / (m_hi - m_lo), 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      issue_one<G, FS>();
      __builtin_amdgcn_sched_barrier(0);
      step<MODE, RS, FS, G + 1>(cf, nf, acc);
    } else {
      if constexpr (RS < 0) next_read_slot();
      __builtin_amdgcn_s_waitcnt(vmcnt_imm(3 * P));
      __builtin_amdgcn_s_barrier();
    }
  }

  // Steps [first, last) in MODE (an even number of them); the fragments of step `first` are in f0 on entry and
  // those of step `last` on exit.  Six steps at a time with the ring slots as immediates when `rd` is at slot
  // 1 and `fill` at slot 5 (true at the first step of a tile), the rest with `rd` / `fill`.
  template <int MODE, bool ALIGNED>
  __device__ __forceinline__ void run(int first, int last, v4i (&f0)[NF], v4i (&f1)[NF], v16f (&acc)[MI][NI]) {
    int j = first;
    if constexpr (ALIGNED) {
      for (; j + 6 <= last; j += 6) {
        step<MODE, 1, 5>(f0, f1, acc);
        step<MODE, 2, 0>(f1, f0, acc);
        step<MODE, 3, 1>(f0, f1, acc);
        step<MODE, 4, 2>(f1, f0, acc);
        step<MODE, 5, 3>(f0, f1, acc);
        step<MODE, 0, 4>(f1, f0, acc);
      }
    }
    for (; j < last; j += 2) {
      step<MODE>(f0, f1, acc);
      step<MODE>(f1, f0, acc);
    }
  }

  __device__ __forceinline__ void drain() const {
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    __syncthreads();
  }
};

struct Fused8Args {
  const uint8_t *xbuf, *wbuf;  // operand buffers (activations, weights), outlier columns included
  const uint16_t *meta, *s_col, *w_red, *bias;
  uint16_t *out;
  int M, N, ldo, K, F;  // N: columns of this launch (s_col, ... start at its first column)
  int n_first;          // first column of this launch inside the weight buffer's row numbering
  int N_total;          // rows of the weight buffer
};

// LDS: the ring, reused as the epilogue's staging area (which is larger than this ring for 256x256 tiles), then
// the per-tile vectors behind both
template <class C>
constexpr int tile8_vectors_offset() {
  constexpr int staging = BlockStore<C, uint16_t>::kBytes * C::MI * C::WAVES;
  return staging > Tile8Pipe<C>::SMEM ? staging : Tile8Pipe<C>::SMEM;
}
template <class C>
constexpr int fused8t_smem() {
  return tile8_vectors_offset<C>() + TileVectors<C>::kBytes;
}

template <class C, bool BF16, bool SPLITK = false>
__device__ __forceinline__ void fused8t_tile(const Fused8Args &p, int tm, int tn, uint8_t *smem, int split = 0,
                                             int tile_id = 0, const SplitK *sk = nullptr) {
  using Pipe = Tile8Pipe<C>;
  const int m0 = tm * C::BM, n0 = tn * C::BN;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;
  const Tile8Layout lx = tile8_layout(p.M, p.K, p.F), lw = tile8_layout(p.N_total, p.K, p.F);
  const TileVectors<C> tv(smem + tile8_vectors_offset<C>());
  for (int i = threadIdx.x; i < C::BN; i += C::kThreads) {
    const int n = n0 + i < p.N ? n0 + i : p.N - 1;
    tv.scol[i] = to_f32<BF16>(p.s_col[n]);
    tv.wred[i] = p.w_red ? to_f32<BF16>(p.w_red[n]) : 0.0f;
    tv.bias[i] = p.bias ? to_f32<BF16>(p.bias[n]) : 0.0f;
  }
  for (int i = threadIdx.x; i < C::BM; i += C::kThreads) {
    const int64_t m = m0 + i < p.M ? m0 + i : p.M - 1;
    // asymmetric: meta holds (scale, zero) pairs; symmetric (no w_red): one scale per row and no zero term
    const float s = to_f32<BF16>(p.meta[p.w_red ? 2 * m : m]);
    tv.srow[i] = s;
    tv.zs[i] = p.w_red ? to_f32<BF16>(p.meta[2 * m + 1]) + 128.0f * s : 0.0f;
  }  // made visible by the first barrier of the pipeline

  v16f acc[C::MI][C::NI];  // integer bit patterns during the first phase, floats afterwards
#pragma unroll
  for (int mi = 0; mi < C::MI; ++mi)
#pragma unroll
    for (int ni = 0; ni < C::NI; ++ni)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0.0f;

  Pipe pipe;
  v4i f0[Pipe::NF], f1[Pipe::NF];
  if constexpr (!SPLITK) {
    pipe.init(smem, p.xbuf, lx, m0 / 64, p.wbuf, lw, (p.n_first + n0) / 64);
    pipe.start();
    pipe.read_all(f0);
    pipe.template run<kInt8, true>(0, pipe.steps0, f0, f1, acc);
  } else {
    const int total = static_cast<int>(lx.steps), k0 = split * sk->per;
    const int k1 = k0 + sk->per < total ? k0 + sk->per : total;
    pipe.init(smem, p.xbuf, lx, m0 / 64, p.wbuf, lw, (p.n_first + n0) / 64, k0, k1 - k0, 0);
    pipe.start();
    pipe.read_all(f0);
    pipe.template run<kInt8, true>(0, pipe.steps0, f0, f1, acc);
    pipe.drain();  // the copies past the last step have landed too: the ring is free
    if (!splitk_combine<C, true>(acc, *sk, tile_id, split, smem)) return;
    if (lx.fsteps > 0) {
      pipe.init(smem, p.xbuf, lx, m0 / 64, p.wbuf, lw, (p.n_first + n0) / 64, total, 0, static_cast<int>(lx.fsteps));
      pipe.start();
      pipe.read_all(f0);
    } else {
      pipe.steps0 = pipe.steps = 0;
    }
  }

  // acc -> f32(acc) * (s_row * s_col) + (zs * w_red + bias), in place, one 32x32 block at a time (the zero-point and
  // bias term is the addend of the multiply: the epilogue only converts and stores)
  float srow[C::MI], zsr[C::MI];
#pragma unroll
  for (int mi = 0; mi < C::MI; ++mi) {
    srow[mi] = tv.srow[wm * C::WM + mi * 32 + (lane & 31)];
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
        const float raw = agpr_read(acc[mi][ni][v]);
        acc[mi][ni][v] = agpr_write(__builtin_fmaf(static_cast<float>(__float_as_int(raw)), srow[mi] * scv[v],
                                                   __builtin_fmaf(zsr[mi], wrv[v], bsv[v])));
      }
    }
  }
  // the fragments in f0 are those of the first outlier step already (same 16-byte reads)
  pipe.template run<BF16 ? kBF16 : kF16, false>(pipe.steps0, pipe.steps, f0, f1, acc);
  pipe.drain();

  // out = storage(acc): all row blocks of the wave staged in the (now idle) ring, read back
  // as whole row segments, stored
  using Store = BlockStore<C, uint16_t>;
  static_assert(Store::kBytes * C::MI * C::WAVES <= tile8_vectors_offset<C>(), "staging ends before the vectors");
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
__global__ __launch_bounds__(C::kThreads) void gemm_fused8t_kernel(Fused8Args p, int tiles_m, int tiles_n) {
  extern __shared__ __align__(16) uint8_t smem[];
  int tm, tn;
  if (!tile_of_block(blockIdx.x, tiles_m, tiles_n, tm, tn)) return;
  fused8t_tile<C, BF16>(p, tm, tn, smem);
}

// K split over sk.splits workgroups per tile: block b works on tile b % grid_tiles (same XCD for all splits of a
// tile's neighbourhood), split b / grid_tiles.
template <class C, bool BF16>
__global__ __launch_bounds__(C::kThreads) void gemm_fused8t_splitk_kernel(Fused8Args p, int tiles_m, int tiles_n,
                                                                           SplitK sk) {
  extern __shared__ __align__(16) uint8_t smem[];
  int tm, tn;
  const int split = blockIdx.x / sk.grid_tiles;
  if (!tile_of_block(blockIdx.x - split * sk.grid_tiles, tiles_m, tiles_n, tm, tn)) return;
  fused8t_tile<C, BF16, true>(p, tm, tn, smem, split, tm * tiles_n + tn, &sk);
}

// One launch, two tile shapes (see gemm_i32_split_kernel).
template <class CW, class CT, bool BF16>
__global__ __launch_bounds__(CW::kThreads) void gemm_fused8t_split_kernel(Fused8Args wide, Fused8Args tail,
                                                                          SplitGrid grid) {
  static_assert(CW::kThreads == CT::kThreads, "one block size");
  extern __shared__ __align__(16) uint8_t smem[];
  int tm, tn;
  const int kind = grid.locate(blockIdx.x, tm, tn);
  if (kind == 1) {
    fused8t_tile<CW, BF16>(wide, tm, tn, smem);
  } else if (kind == 2) {
    fused8t_tile<CT, BF16>(tail, tm, tn, smem);
  }
}

}  // namespace quik
