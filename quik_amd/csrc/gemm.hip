// Host side of the GEMM entry points: argument checks, tile planning, launches.
// The kernels live in gemm_kernels.h.
#include <atomic>
#include <cstdint>
#include <mutex>

#include "colmap.h"
#include "gemm_decode.h"
#include "gemm_gemv.h"
#ifndef GEMV_MAX_ROWS
#define GEMV_MAX_ROWS 2
#endif
#include "gemm_tile8.h"
#include "gemm_kernels.h"

namespace quik {
namespace {

// Tile configurations.  "dma" ones use the direct-to-LDS pipelined main loop and need K bytes
// (and outlier bytes) per row to be a multiple of 64; the plain ones accept anything.
using CfgL = Cfg<256, 256, 2, 2, 2>;   // prefill: 128x128 per wave, 256 accumulator registers
using CfgH = Cfg<256, 128, 2, 2, 2>;   // half-width tile that evens out the last round
using CfgM = Cfg<128, 128, 2, 2, 2>;   // mid-size problems, two workgroups per CU
using CfgN = Cfg<128, 64, 2, 2, 2>;    // few tiles: narrower ones put more CUs to work, three workgroups per CU
using CfgN6 = Cfg<128, 64, 2, 2, 2>;   // 6-bit path, 86 .. ~150 tiles of 128x128 and no K split: twice as many workgroups
using CfgL8 = Cfg<256, 256, 2, 4, 2>;  // 6-bit path, launches of 256x256 tiles only: two waves per SIMD (1-5 % faster than CfgL)
using CfgLp = Cfg<256, 256, 2, 2, 0>;  // plain fallbacks
using CfgMp = Cfg<128, 128, 2, 2, 0>;

constexpr int kMaxCUs = 256;  // MI355X; sizes the static K-split scratch array

// Zero-fill of a few words by a kernel: the arrival counters of the K split are cleared with it, not with
// hipMemsetAsync, because the caller's stream may be under capture and a memset node in a captured graph is not
// reliable on replays.
__global__ __launch_bounds__(256) void clear_words_kernel(uint32_t *p, int words) {
  for (int i = blockIdx.x * 256 + threadIdx.x; i < words; i += gridDim.x * 256) p[i] = 0u;
}
constexpr int kLdsBytes = 160 * 1024;  // per CU, and the most one workgroup may ask for

// Kernels that ask for more than 48 KB of dynamic LDS need the attribute raised once per device; the (kernel,
// device) pairs already done are remembered, so a launch costs a table look-up, not a runtime call.
struct PreparedKernels {
  static constexpr int kSlots = 512;  // open addressing; far more than the instantiations in this file
  std::atomic<uintptr_t> key[kSlots];
  bool seen_or_insert(uintptr_t k, bool insert) {
    for (int i = 0, h = static_cast<int>((k >> 4) % kSlots); i < kSlots; ++i, h = (h + 1) % kSlots) {
      uintptr_t cur = key[h].load(std::memory_order_acquire);
      if (cur == k) return true;
      if (cur == 0) {
        if (!insert) return false;
        if (key[h].compare_exchange_strong(cur, k, std::memory_order_acq_rel) || cur == k) return true;
      }
    }
    return false;
  }
};
PreparedKernels g_prepared;

template <typename K>
int prepare(K kern, int smem) {
  if (smem > 48 * 1024) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
      set_last_hip_error(e);
      return QUIK_ERR_LAUNCH;
    }
    // kernel entry addresses are at least 16-byte aligned: the low bits carry the device, bit 0 marks a used slot
    const uintptr_t k = (reinterpret_cast<uintptr_t>(kern) << 8) | (static_cast<uintptr_t>(dev & 0x7F) << 1) | 1u;
    if (g_prepared.seen_or_insert(k, false)) return QUIK_OK;
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) {
      set_last_hip_error(e);
      return QUIK_ERR_LAUNCH;
    }
    g_prepared.seen_or_insert(k, true);
  }
  return QUIK_OK;
}

template <class C>
int grid_of(int64_t M, int64_t N, int &tiles_m, int &tiles_n) {
  tiles_m = static_cast<int>((M + C::BM - 1) / C::BM);
  tiles_n = static_cast<int>((N + C::BN - 1) / C::BN);
  return static_cast<int>(((int64_t(tiles_m) * tiles_n + 7) / 8) * 8);
}

template <class C, int MODE>
int launch_i32(const I32Args &a, hipStream_t st) {
  if (a.N <= 0) return QUIK_OK;
  int tiles_m, tiles_n;
  const int grid = grid_of<C>(a.M, a.N, tiles_m, tiles_n);
  auto kern = gemm_i32_kernel<C, MODE>;
  if (int rc = prepare(kern, C::SMEM)) return rc;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(C::kThreads), C::SMEM, st, a, tiles_m, tiles_n);
  return check_launch();
}

// Workgroup id layout of a two-shape launch: half of the narrow tiles (at most half a round) lead.
template <class CW, class CT>
SplitGrid split_grid(int64_t M, int64_t n_wide, int64_t n_tail, int &tail_blocks) {
  SplitGrid g;
  g.wide_blocks = grid_of<CW>(M, n_wide, g.tiles_m, g.tiles_n_wide);
  tail_blocks = grid_of<CT>(M, n_tail, g.tiles_m, g.tiles_n_tail);
  int lead = (tail_blocks / 2) & ~7;
  if (lead > num_cus() / 2) lead = num_cus() / 2;
  g.lead = lead;
  return g;
}

template <class CW, class CT, int MODE>
int launch_i32_split(const I32Args &wide, const I32Args &tail, hipStream_t st) {
  if (wide.N <= 0) return launch_i32<CT, MODE>(tail, st);
  if (tail.N <= 0) return launch_i32<CW, MODE>(wide, st);
  int tail_blocks;
  const SplitGrid grid = split_grid<CW, CT>(wide.M, wide.N, tail.N, tail_blocks);
  auto kern = gemm_i32_split_kernel<CW, CT, MODE>;
  constexpr int smem = CW::SMEM > CT::SMEM ? CW::SMEM : CT::SMEM;
  if (int rc = prepare(kern, smem)) return rc;
  hipLaunchKernelGGL(kern, dim3(grid.wide_blocks + tail_blocks), dim3(CW::kThreads), smem, st, wide, tail, grid);
  return check_launch();
}

template <class C, int MODE, bool BF16>
int launch_fused(const FusedArgs &p, hipStream_t st) {
  if (p.N <= 0) return QUIK_OK;
  int tiles_m, tiles_n;
  const int grid = grid_of<C>(p.M, p.N, tiles_m, tiles_n);
  auto kern = gemm_fused_kernel<C, MODE, BF16>;
  constexpr int smem = fused_smem<C>();
  if (int rc = prepare(kern, smem)) return rc;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(C::kThreads), smem, st, p, tiles_m, tiles_n);
  return check_launch();
}

template <class CW, class CT, int MODE, bool BF16>
int launch_fused_split(const FusedArgs &wide, const FusedArgs &tail, hipStream_t st) {
  if (wide.N <= 0) return launch_fused<CT, MODE, BF16>(tail, st);
  if (tail.N <= 0) return launch_fused<CW, MODE, BF16>(wide, st);
  int tail_blocks;
  const SplitGrid grid = split_grid<CW, CT>(wide.M, wide.N, tail.N, tail_blocks);
  auto kern = gemm_fused_split_kernel<CW, CT, MODE, BF16>;
  constexpr int smem = fused_smem<CW>() > fused_smem<CT>() ? fused_smem<CW>() : fused_smem<CT>();
  if (int rc = prepare(kern, smem)) return rc;
  hipLaunchKernelGGL(kern, dim3(grid.wide_blocks + tail_blocks), dim3(CW::kThreads), smem, st, wide, tail, grid);
  return check_launch();
}

// M <= 32: the weight-streaming kernel of gemm_decode.h.  8 waves per 32-column slab when there are few
// slabs (so that enough loads are in flight chip-wide) and K gives every wave at least two 128-byte
// chunks per row; otherwise 4 waves, which lets two workgroups share a CU.
int decode_waves(int64_t N, int64_t kbytes) {
  const int64_t slabs = (N + 31) / 32, chunks = (kbytes + kDecodeChunk - 1) / kDecodeChunk;
  return (chunks >= 16 && slabs <= num_cus()) ? 8 : 4;
}

template <int MODE, bool BF16, bool FUSED, int WAVES, bool XLDS>
int launch_decode_w(const FusedArgs &p, int32_t *C, int ldc, hipStream_t st) {
  auto kern = gemm_decode_kernel<MODE, BF16, FUSED, WAVES, XLDS>;
  const int smem = decode_smem<WAVES, FUSED, XLDS>() + (XLDS ? static_cast<int>(decode_x_lds_bytes(p.M, p.kbytes)) : 0);
  // XLDS: the LDS size varies from call to call with the row count, and prepare() sets the attribute once per
  // kernel and device: set it to the most any call may ask for
  if (int rc = prepare(kern, XLDS ? kLdsBytes : smem)) return rc;
  // persistent workgroups: as many as are resident at once (8 waves per CU at this register count; the LDS copy
  // of the token rows leaves room for one workgroup)
  // Every workgroup walks the same number of slabs (one more or less): with 896 slabs, 224 workgroups of 4 slabs
  // finish when 256 workgroups of 3 or 4 do, and share the memory system among fewer.
  const int64_t slabs = (p.N + 31) / 32, resident = int64_t(num_cus()) * (XLDS ? 1 : 8 / WAVES);
  const int64_t per = (slabs + resident - 1) / resident, grid = (slabs + per - 1) / per;
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(grid)), dim3(WAVES * 64), smem, st, p, C, ldc);
  return check_launch();
}

// The token rows stay in LDS when they fit beside the reduction area and there is more than one slab per
// workgroup to reuse them for (with fewer than 4 rows the L2 reads they replace cost less than the copy).
template <int WAVES, bool FUSED>
bool decode_x_fits(const FusedArgs &p) {
  return p.M >= 4 && decode_smem<WAVES, FUSED, true>() + decode_x_lds_bytes(p.M, p.kbytes) <= kLdsBytes &&
         (p.N + 31) / 32 > num_cus();
}

// At most kGemvMaxRows token rows (fused form): one wave per output column, gemm_gemv.h.  Needs 16-byte aligned rows
// of both weight arrays and room in LDS for the token rows.
constexpr int kGemvMaxRows = GEMV_MAX_ROWS;
bool gemv_ok(const FusedArgs &p, bool quant = false) {
  const auto aligned = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  const int mt = p.M <= 1 ? 1 : p.M <= 2 ? 2 : 4;
  return p.M >= 1 && p.M <= kGemvMaxRows && p.kbytes >= 16 && p.kbytes % 16 == 0 && p.F % 8 == 0 &&
         (quant || aligned(p.qx)) && aligned(p.qw) && (p.F == 0 || ((quant || aligned(p.fp_x)) && aligned(p.fp_w))) &&
         gemv_smem(mt, p.kbytes, p.F) + gemv_table_bytes((p.N + kGemvWaves * num_cus() - 1) / (kGemvWaves * num_cus())) <=
             kLdsBytes;
}
template <int MODE, bool BF16, int MT, int QUANT>
int launch_gemv_mt(const FusedArgs &p, const GemvQuant &q, hipStream_t st) {
  auto kern = gemv_decode_kernel<MODE, BF16, MT, QUANT>;
  if (int rc = prepare(kern, kLdsBytes)) return rc;  // (the size varies with the layer: set once to the most)
  // persistent waves, one column at a time each: two workgroups per CU when their LDS fits twice
  const int64_t fixed = gemv_smem(MT, p.kbytes, p.F) + (QUANT != kGemvNoQuant ? gemv_quant_lds(q.cols, q.num_int).bytes : 0);
  const int64_t per_cu = 2 * (fixed + 4096) <= kLdsBytes ? 2 : 1;
  int64_t grid = (p.N + kGemvWaves - 1) / kGemvWaves;
  if (grid > per_cu * num_cus()) grid = per_cu * num_cus();
  const int64_t smem = fixed + gemv_table_bytes((p.N + kGemvWaves * grid - 1) / (kGemvWaves * grid));
  if (smem > kLdsBytes) return kChainNotHandled;
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(grid)), dim3(kGemvWaves * 64), static_cast<size_t>(smem), st, p, q);
  return check_launch();
}
template <int MODE, bool BF16, int QUANT = kGemvNoQuant>
int launch_gemv(const FusedArgs &p, const GemvQuant &q, hipStream_t st) {
  if (p.M <= 1) return launch_gemv_mt<MODE, BF16, 1, QUANT>(p, q, st);
  if constexpr (kGemvMaxRows > 2) {  // (only built when the row limit is raised: gemv_ok() admits no such call otherwise)
    if (p.M > 2) return launch_gemv_mt<MODE, BF16, 4, QUANT>(p, q, st);
  }
  return launch_gemv_mt<MODE, BF16, 2, QUANT>(p, q, st);
}

template <int MODE, bool BF16, bool FUSED>
int launch_decode(const FusedArgs &p, int32_t *C, int ldc, hipStream_t st) {
  if constexpr (FUSED) {
    if (gemv_ok(p)) {
      const int rc = launch_gemv<MODE, BF16>(p, GemvQuant{}, st);
      if (rc != kChainNotHandled) return rc;
    }
  }
  if (decode_x_fits<8, FUSED>(p)) return launch_decode_w<MODE, BF16, FUSED, 8, true>(p, C, ldc, st);
  if (decode_waves(p.N, p.kbytes) == 8) return launch_decode_w<MODE, BF16, FUSED, 8, false>(p, C, ldc, st);
  return launch_decode_w<MODE, BF16, FUSED, 4, false>(p, C, ldc, st);
}

// How a problem is cut into tiles.  Columns [0, n_wide) go to 256x256 tiles, [n_wide, N) to
// 256x128 tiles, all in one launch with the wide tiles first.  One workgroup fits per CU and the
// hardware hands the next workgroup to whichever CU frees up, so the run time is the makespan of
// that list schedule; the narrow tiles even out its end.
struct Plan {
  enum Kind { kSmall, kMid, kNarrow, kMidPlain, kLargePlain, kSplit } kind;
  int64_t n_wide;
};

// relative tile costs in percent of a 256x256 tile (measured)
constexpr int kCostWide = 100, kCostHalf = 55, kCostMid = 28;

// Makespan of `wide` tiles followed by `half` tiles on the GPU's CUs under greedy list scheduling.
int64_t makespan(int64_t wide, int64_t half, int cost_half = kCostHalf) {
  // after the wide tiles: `rem` CUs carry one tile more than the others
  const int64_t full = wide / num_cus(), rem = wide % num_cus();
  int64_t lo_level = full * kCostWide, lo_count = num_cus() - rem;  // less loaded CUs
  int64_t hi_level = lo_level + kCostWide, hi_count = rem;
  // the half tiles go to the least loaded CUs, a whole level at a time
  while (half > 0) {
    if (hi_count == 0 || lo_level + cost_half <= hi_level) {
      if (half >= lo_count && lo_level + cost_half < hi_level && hi_count > 0) {
        lo_level += cost_half;
        half -= lo_count;
      } else if (hi_count == 0) {
        const int64_t rounds = half / lo_count, left = half % lo_count;
        return lo_level + rounds * cost_half + (left ? cost_half : 0);
      } else if (half >= lo_count) {  // lo reaches hi's level exactly
        lo_level += cost_half;
        half -= lo_count;
        if (lo_level == hi_level) {
          lo_count += hi_count;
          hi_count = 0;
        }
      } else {
        const int64_t top = lo_level + cost_half;
        return top > hi_level ? top : hi_level;
      }
    } else {
      // adding a half tile to the lower level overtakes the higher one: swap roles afterwards
      if (half >= lo_count) {
        half -= lo_count;
        const int64_t new_hi = lo_level + cost_half, new_hi_count = lo_count;
        lo_level = hi_level;
        lo_count = hi_count;
        hi_level = new_hi;
        hi_count = new_hi_count;
      } else {
        return lo_level + cost_half;
      }
    }
  }
  return hi_count > 0 ? hi_level : lo_level;
}

Plan make_plan(int64_t M, int64_t N, bool dma_ok) {
  if (M <= 32) return {Plan::kSmall, 0};
  const int64_t tiles_m = (M + 255) / 256;
  auto rounds = [](int64_t tiles) { return (tiles + num_cus() - 1) / num_cus(); };
  if (!dma_ok) {
    if (M <= 128 || tiles_m * ((N + 255) / 256) < num_cus() / 2) return {Plan::kMidPlain, 0};
    return {Plan::kLargePlain, 0};
  }
  const int64_t mid = rounds(((M + 127) / 128) * ((N + 127) / 128)) * kCostMid;
  int64_t best = INT64_MAX, best_n = 0;
  for (int64_t n_wide = 0; n_wide <= N; n_wide += 256) {
    const int64_t c = makespan(tiles_m * (n_wide / 256), tiles_m * ((N - n_wide + 127) / 128));
    if (c <= best) {
      best = c;
      best_n = n_wide;
    }
  }
  if (M <= 128 || mid < best) {
    // with few 128x128 tiles most CUs would idle: 128x64 tiles put twice as many to work
    // (measured: 15-20 % less time up to about 130 tiles, no gain at 224)
    const int64_t mid_tiles = ((M + 127) / 128) * ((N + 127) / 128);
    return {mid_tiles <= 160 ? Plan::kNarrow : Plan::kMid, 0};
  }
  return {Plan::kSplit, best_n};
}

int check_gemm_args(const void *A, const void *B, const void *C, int64_t M, int64_t N, int64_t K, int bits) {
  if (M < 0 || N < 0 || K <= 0) return QUIK_ERR_SHAPE;
  if (M == 0 || N == 0) return QUIK_OK;
  if (!A || !B || !C) return QUIK_ERR_NULL;
  if (bits == 4 ? (K % 32 != 0) : (K % 16 != 0)) return QUIK_ERR_ALIGN;
  auto misaligned = [](const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 != 0; };
  if (misaligned(A) || misaligned(B)) return QUIK_ERR_ALIGN;
  if (M > (1 << 30) || N > (1 << 30) || K > (int64_t(1) << 30)) return QUIK_ERR_RANGE;
  if (bits == 4 && K >= 131072) return QUIK_ERR_RANGE;
  return QUIK_OK;
}

template <int MODE>
int run_i32(const uint8_t *X, const uint8_t *W, int32_t *C, int64_t M, int64_t N, int64_t kbytes, hipStream_t st) {
  I32Args a{X, W, C, static_cast<int>(M), static_cast<int>(N), static_cast<int>(N), static_cast<int>(kbytes)};
  const Plan plan = make_plan(M, N, kbytes % 64 == 0);
  switch (plan.kind) {
    case Plan::kSmall: {
      FusedArgs p{};
      p.qx = X;
      p.qw = W;
      p.M = a.M;
      p.N = a.N;
      p.kbytes = a.kbytes;
      return launch_decode<MODE, false, false>(p, C, a.ldc, st);
    }
    case Plan::kMid: return launch_i32<CfgM, MODE>(a, st);
    case Plan::kNarrow: return launch_i32<CfgN, MODE>(a, st);
    case Plan::kMidPlain: return launch_i32<CfgMp, MODE>(a, st);
    case Plan::kLargePlain: return launch_i32<CfgLp, MODE>(a, st);
    default: break;
  }
  I32Args wide = a, tail = a;
  wide.N = static_cast<int>(plan.n_wide);
  tail.N = static_cast<int>(N - plan.n_wide);
  tail.W = W + plan.n_wide * kbytes;
  tail.C = C + plan.n_wide;
  return launch_i32_split<CfgL, CfgH, MODE>(wide, tail, st);
}

template <class C, int MODE, bool ASYM>
int launch_chain(const I32Args &a, const ChainArgs &e, hipStream_t st) {
  int tiles_m, tiles_n;
  const int grid = grid_of<C>(a.M, a.N, tiles_m, tiles_n);
  auto kern = gemm_chain_kernel<C, MODE, ASYM>;
  if (int rc = prepare(kern, C::SMEM)) return rc;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(C::kThreads), C::SMEM, st, a, e, tiles_m, tiles_n);
  return check_launch();
}

template <int MODE, bool ASYM>
int run_chain(const I32Args &a, const ChainArgs &e, hipStream_t st) {
  switch (make_plan(a.M, a.N, a.kbytes % 64 == 0).kind) {
    case Plan::kSmall: return kChainNotHandled;  // at most 32 rows: the weight-streaming kernel has no such epilogue
    case Plan::kMid: return launch_chain<CfgM, MODE, ASYM>(a, e, st);
    case Plan::kNarrow: return launch_chain<CfgN, MODE, ASYM>(a, e, st);
    case Plan::kMidPlain:
    case Plan::kLargePlain: return launch_chain<CfgMp, MODE, ASYM>(a, e, st);
    default: return launch_chain<CfgL, MODE, ASYM>(a, e, st);
  }
}

// Tile plan of the 6-bit path (gemm_fp6.h).  Costs in percent of a 256x256 tile, measured at K = 7936, F = 256:
// a 256x128 tile 59; 128x128 tiles run two to a CU, 66 for a pair, 36 for one that has the CU to itself.
Plan make_plan6(int64_t M, int64_t N, int64_t min_rows) {
  if (M < min_rows) return {Plan::kSmall, 0};
  const int64_t tiles_m = (M + 255) / 256;
  const int64_t mid_tiles = ((M + 127) / 128) * ((N + 127) / 128);
  const int64_t pairs = mid_tiles / (2 * num_cus()), left = mid_tiles % (2 * num_cus());
  const int64_t mid = pairs * 66 + (left == 0 ? 0 : left <= num_cus() ? 36 : 66);
  int64_t best = INT64_MAX, best_n = 0;
  for (int64_t n_wide = 0; n_wide <= N + 255; n_wide += 256) {
    const int64_t nw = n_wide < N ? n_wide : N;   // the last candidate: wide tiles only, the last one ragged
    const int64_t c = makespan(tiles_m * ((nw + 255) / 256), tiles_m * ((N - nw + 127) / 128), 59);
    if (c <= best) {
      best = c;
      best_n = nw;
    }
  }
  if (mid < best) return {Plan::kMid, 0};
  return {Plan::kSplit, best_n};
}

// Split over K for the tile-ordered kernels: few 128x128 tiles (at most half the CUs) and a long K.  Each of
// `splits` workgroups per tile takes `per` steps (even); workspace = counters (one per tile, zero between launches)
// followed by the partial accumulators.
constexpr int64_t kSplitCounterBytes = 4096;
constexpr int64_t kSplitMinSteps8 = 32, kSplitMinSteps6 = 32;  // at least 1024 (int8) / 2048 (6-bit) elements of K per workgroup
struct SplitPlan {
  int splits, per;
  int64_t bytes;
};
// min_splits: with two workgroups per tile the exchange and the restart for the outlier steps cost the 6-bit path
// (K <= 8192 in every Llama layer it serves) what the halved K loop saves; measured gains start at three.
SplitPlan plan_splitk(int64_t M, int64_t N, int64_t steps, int64_t min_steps, int64_t min_rows, int64_t min_splits) {
  SplitPlan none{1, 0, 0};
  if (make_plan6(M, N, min_rows).kind != Plan::kMid) return none;
  const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
  if (tiles > num_cus() / 2 || tiles * 4 > kSplitCounterBytes) return none;
  for (int64_t splits = num_cus() / tiles < 8 ? num_cus() / tiles : 8; splits >= min_splits; --splits) {
    const int64_t per = ((steps + splits - 1) / splits + 1) / 2 * 2;
    if (per >= min_steps && (splits - 1) * per < steps)
      return {static_cast<int>(splits), static_cast<int>(per), kSplitCounterBytes + tiles * splits * 128 * 128 * 4};
  }
  return none;
}

// The arrival counters are zero between launches because every launch that completes returns them there.  After a
// launch that was refused nothing ran, but the caller may not know how far an earlier one got: clear the counters
// behind a failed launch so that the next one on this workspace starts clean.
int splitk_launch_status(void *workspace, hipStream_t st) {
  const int rc = check_launch();
  if (rc != QUIK_OK) {
    hipLaunchKernelGGL(clear_words_kernel, dim3(static_cast<unsigned>(kSplitCounterBytes / 4 / 256)), dim3(256), 0, st,
                       static_cast<uint32_t *>(workspace), static_cast<int>(kSplitCounterBytes / 4));
    (void)hipGetLastError();  // the status reported is that of the launch that failed
  }
  return rc;
}

template <bool BF16>
int launch_fused6_splitk(const Fused6Args &p, const SplitPlan &sp, void *workspace, hipStream_t st) {
  int tiles_m, tiles_n;
  const int grid_tiles = grid_of<CfgM>(p.M, p.N, tiles_m, tiles_n);
  SplitK sk{sp.splits, sp.per, grid_tiles, static_cast<uint32_t *>(workspace),
            reinterpret_cast<int32_t *>(static_cast<uint8_t *>(workspace) + kSplitCounterBytes)};
  auto kern = gemm_fused6_splitk_kernel<CfgM, BF16>;
  constexpr int smem = fused6_smem<CfgM>();
  if (int rc = prepare(kern, smem)) return rc;
  hipLaunchKernelGGL(kern, dim3(grid_tiles * sp.splits), dim3(CfgM::kThreads), smem, st, p, tiles_m, tiles_n, sk);
  return splitk_launch_status(workspace, st);
}

template <bool BF16>
int launch_fused8t_splitk(const Fused8Args &p, const SplitPlan &sp, void *workspace, hipStream_t st) {
  int tiles_m, tiles_n;
  const int grid_tiles = grid_of<CfgM>(p.M, p.N, tiles_m, tiles_n);
  SplitK sk{sp.splits, sp.per, grid_tiles, static_cast<uint32_t *>(workspace),
            reinterpret_cast<int32_t *>(static_cast<uint8_t *>(workspace) + kSplitCounterBytes)};
  auto kern = gemm_fused8t_splitk_kernel<CfgM, BF16>;
  constexpr int smem = fused8t_smem<CfgM>();
  if (int rc = prepare(kern, smem)) return rc;
  hipLaunchKernelGGL(kern, dim3(grid_tiles * sp.splits), dim3(CfgM::kThreads), smem, st, p, tiles_m, tiles_n, sk);
  return splitk_launch_status(workspace, st);
}

template <class C, bool BF16>
int launch_fused6(const Fused6Args &p, hipStream_t st) {
  if (p.N <= 0) return QUIK_OK;
  int tiles_m, tiles_n;
  const int grid = grid_of<C>(p.M, p.N, tiles_m, tiles_n);
  auto kern = gemm_fused6_kernel<C, BF16>;
  constexpr int smem = fused6_smem<C>();
  if (int rc = prepare(kern, smem)) return rc;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(C::kThreads), smem, st, p, tiles_m, tiles_n);
  return check_launch();
}

template <class CW, class CT, bool BF16>
int launch_fused6_split(const Fused6Args &wide, const Fused6Args &tail, hipStream_t st) {
  if (wide.N <= 0) return launch_fused6<CT, BF16>(tail, st);
  if (tail.N <= 0) return launch_fused6<CW, BF16>(wide, st);
  int tail_blocks;
  SplitGrid grid = split_grid<CW, CT>(wide.M, wide.N, tail.N, tail_blocks);
  grid.lead = 0;  // this kernel lives on L2 hits between the tiles of an XCD that share operand rows: keep them in step
  auto kern = gemm_fused6_split_kernel<CW, CT, BF16>;
  constexpr int smem = fused6_smem<CW>() > fused6_smem<CT>() ? fused6_smem<CW>() : fused6_smem<CT>();
  if (int rc = prepare(kern, smem)) return rc;
  hipLaunchKernelGGL(kern, dim3(grid.wide_blocks + tail_blocks), dim3(CW::kThreads), smem, st, wide, tail, grid);
  return check_launch();
}

// The 6-bit matrix-core path (gemm_fp6.h): 256x256 tiles alone (eight waves), 256x256 + 256x128 tiles in one
// launch (four waves), or 128x128 tiles.
template <bool BF16>
int run_fused6(const Fused6Args &p, hipStream_t st, void *workspace, int64_t workspace_bytes) {
  // any row count: up to 32 rows the weight-streaming kernel on the packed nibbles reads a third fewer bytes, and
  // callers that keep both weight copies route such calls there
  const Plan plan = make_plan6(p.M, p.N, 1);
  if (plan.kind == Plan::kSplit && plan.n_wide >= p.N) return launch_fused6<CfgL8, BF16>(p, st);
  if (plan.kind != Plan::kSplit) {
    const SplitPlan sp = plan_splitk(p.M, p.N, p.K / 64, kSplitMinSteps6, 1, 3);
    if (sp.splits > 1 && workspace && workspace_bytes >= sp.bytes) return launch_fused6_splitk<BF16>(p, sp, workspace, st);
    // too few 128x128 tiles for the CUs and no K split (it takes three workgroups per tile to pay): 128x64 tiles
    const int64_t mid_tiles = ((p.M + 127) / 128) * ((p.N + 127) / 128);
    // (up to 0.62 tiles per CU: measured 6 - 12 % less time on 13B gate_proj at 128 tokens, 70B k_proj and the
    // 512 x 4096 x 4096 configuration; with 0.88 tiles per CU, 70B gate_proj at 64 tokens, 11 % more)
    if (mid_tiles * 8 <= int64_t(num_cus()) * 5) return launch_fused6<CfgN6, BF16>(p, st);
    return launch_fused6<CfgM, BF16>(p, st);
  }
  Fused6Args wide = p, tail = p;
  const int64_t nw = plan.n_wide;
  wide.N = static_cast<int>(nw);
  tail.N = static_cast<int>(p.N - nw);
  tail.n_first = static_cast<int>(nw);
  tail.s_col = p.s_col + nw;
  tail.w_red = p.w_red ? p.w_red + nw : nullptr;
  tail.bias = p.bias ? p.bias + nw : nullptr;
  tail.out = p.out + nw;
  return launch_fused6_split<CfgL, CfgH, BF16>(wide, tail, st);
}

template <class C, bool BF16>
int launch_fused8t(const Fused8Args &p, hipStream_t st) {
  if (p.N <= 0) return QUIK_OK;
  int tiles_m, tiles_n;
  const int grid = grid_of<C>(p.M, p.N, tiles_m, tiles_n);
  auto kern = gemm_fused8t_kernel<C, BF16>;
  constexpr int smem = fused8t_smem<C>();
  if (int rc = prepare(kern, smem)) return rc;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(C::kThreads), smem, st, p, tiles_m, tiles_n);
  return check_launch();
}

template <class CW, class CT, bool BF16>
int launch_fused8t_split(const Fused8Args &wide, const Fused8Args &tail, hipStream_t st) {
  if (wide.N <= 0) return launch_fused8t<CT, BF16>(tail, st);
  if (tail.N <= 0) return launch_fused8t<CW, BF16>(wide, st);
  int tail_blocks;
  SplitGrid grid = split_grid<CW, CT>(wide.M, wide.N, tail.N, tail_blocks);
  grid.lead = 0;  // tiles of an XCD that share operand rows stay in step (L2 hits)
  auto kern = gemm_fused8t_split_kernel<CW, CT, BF16>;
  constexpr int smem = fused8t_smem<CW>() > fused8t_smem<CT>() ? fused8t_smem<CW>() : fused8t_smem<CT>();
  if (int rc = prepare(kern, smem)) return rc;
  hipLaunchKernelGGL(kern, dim3(grid.wide_blocks + tail_blocks), dim3(CW::kThreads), smem, st, wide, tail, grid);
  return check_launch();
}

// W8A8 on tile-ordered operands (gemm_tile8.h): same plan and tile shapes as the 6-bit path.
template <bool BF16>
int run_fused8t(const Fused8Args &p, hipStream_t st, void *workspace, int64_t workspace_bytes) {
  const Plan plan = make_plan6(p.M, p.N, 1);  // any row count: with few rows this path competes with the weight-streaming kernel
  if (plan.kind != Plan::kSplit) {
    const SplitPlan sp = plan_splitk(p.M, p.N, p.K / 32, kSplitMinSteps8, 1, 2);
    if (sp.splits > 1 && workspace && workspace_bytes >= sp.bytes) return launch_fused8t_splitk<BF16>(p, sp, workspace, st);
    return launch_fused8t<CfgM, BF16>(p, st);
  }
  if (plan.n_wide >= p.N) return launch_fused8t<CfgL8, BF16>(p, st);
  Fused8Args wide = p, tail = p;
  const int64_t nw = plan.n_wide;
  wide.N = static_cast<int>(nw);
  tail.N = static_cast<int>(p.N - nw);
  tail.n_first = static_cast<int>(nw);
  tail.s_col = p.s_col + nw;
  tail.w_red = p.w_red ? p.w_red + nw : nullptr;
  tail.bias = p.bias ? p.bias + nw : nullptr;
  tail.out = p.out + nw;
  return launch_fused8t_split<CfgL, CfgH, BF16>(wide, tail, st);
}

template <int MODE, bool BF16>
int run_fused(const FusedArgs &p, hipStream_t st) {
  const Plan plan = make_plan(p.M, p.N, p.kbytes % 64 == 0 && (p.F * 2) % 64 == 0);
  switch (plan.kind) {
    case Plan::kSmall: return launch_decode<MODE, BF16, true>(p, nullptr, 0, st);
    case Plan::kMid: return launch_fused<CfgM, MODE, BF16>(p, st);
    case Plan::kNarrow: return launch_fused<CfgN, MODE, BF16>(p, st);
    case Plan::kMidPlain: return launch_fused<CfgMp, MODE, BF16>(p, st);
    case Plan::kLargePlain: return launch_fused<CfgLp, MODE, BF16>(p, st);
    default: break;
  }
  FusedArgs wide = p, tail = p;
  const int64_t nw = plan.n_wide;
  wide.N = static_cast<int>(nw);
  tail.N = static_cast<int>(p.N - nw);
  tail.qw = p.qw + nw * p.kbytes;
  tail.s_col = p.s_col + nw;
  tail.w_red = p.w_red ? p.w_red + nw : nullptr;
  tail.bias = p.bias ? p.bias + nw : nullptr;
  tail.fp_w = p.fp_w ? p.fp_w + nw * p.F : nullptr;
  tail.out = p.out + nw;
  return launch_fused_split<CfgL, CfgH, MODE, BF16>(wide, tail, st);
}

}  // namespace

// Integer GEMM with the fp16-arithmetic epilogue of the reference's fused ops in one launch (see ChainArgs in
// gemm_kernels.h); kChainNotHandled when the shape belongs to the weight-streaming kernel (at most 32 rows), which
// has no such epilogue: the caller then runs the product and the epilogue as two launches.
int int_gemm_chain(const void *A, const void *B, const void *s_row, const void *s_col, const void *zero_row,
                   const void *w_red, uint16_t shift_bits, const void *y, int64_t M, int64_t N, int64_t K, int bits,
                   void *out, hipStream_t st) {
  if (int rc = check_gemm_args(A, B, out, M, N, K, bits)) return rc;
  I32Args a{static_cast<const uint8_t *>(A), static_cast<const uint8_t *>(B), nullptr, static_cast<int>(M),
            static_cast<int>(N), static_cast<int>(N), static_cast<int>(bits == 4 ? K / 2 : K)};
  ChainArgs e{static_cast<const uint16_t *>(s_row), static_cast<const uint16_t *>(s_col),
              static_cast<const uint16_t *>(zero_row), static_cast<const uint16_t *>(w_red),
              static_cast<const uint16_t *>(y), static_cast<uint16_t *>(out), static_cast<int>(N), shift_bits};
  const bool asym = zero_row != nullptr;
  if (bits == 4) return asym ? run_chain<kInt4, true>(a, e, st) : run_chain<kInt4, false>(a, e, st);
  return asym ? run_chain<kInt8, true>(a, e, st) : run_chain<kInt8, false>(a, e, st);
}
}  // namespace quik

using namespace quik;

extern "C" int quik_int4_matmul(const uint8_t *A, const uint8_t *B, int32_t *C, int64_t M, int64_t N, int64_t K,
                                void *stream) {
  if (int rc = check_gemm_args(A, B, C, M, N, K, 4)) return rc;
  if (M == 0 || N == 0) return QUIK_OK;
  return run_i32<kInt4>(A, B, C, M, N, K / 2, as_stream(stream));
}

extern "C" int quik_int8_matmul(const int8_t *A, const int8_t *B, int32_t *C, int64_t M, int64_t N, int64_t K,
                                void *stream) {
  if (int rc = check_gemm_args(A, B, C, M, N, K, 8)) return rc;
  if (M == 0 || N == 0) return QUIK_OK;
  return run_i32<kInt8>(reinterpret_cast<const uint8_t *>(A), reinterpret_cast<const uint8_t *>(B), C, M, N, K,
                        as_stream(stream));
}

// MixedQLinear forward for at most kGemvMaxRows token rows in ONE launch: the kernel of gemm_gemv.h quantises the
// rows itself (asymmetric activations, or symmetric ones when w_red is NULL: fp16 only, scale = max |x| /
// sym_divisor).  kChainNotHandled: the shape is left to the two-launch path.
int quik::gemv_forward_one_launch(const void *x, int dtype, int64_t rows, int64_t cols, const void *colmap,
                                  int64_t num_int, int64_t num_fp, int bits, const void *qw, const void *s_col,
                                  const void *w_red, const void *fp_w, const void *bias, int64_t N, void *out,
                                  float sym_divisor, hipStream_t st) {
  const bool sym = w_red == nullptr;
  // (cols % 32, num_int % 128: the column map's group and unit tables arrive as whole 16-byte pieces)
  if (rows < 1 || rows > kGemvMaxRows || (sym && dtype != QUIK_F16) || cols % 32 != 0 || cols > kStreamMaxCols || num_int % 128 != 0 ||
      num_fp > kGemvWaves * 64 ||
      (reinterpret_cast<uintptr_t>(x) & 15) != 0 || N > (1 << 30))
    return kChainNotHandled;
  uint32_t words[4];
  if (int rc = colmap_words(colmap, cols, num_int, num_fp, st, words)) return rc == QUIK_ERR_COLMAP ? kChainNotHandled : rc;
  if (!(words[0] & kColmapStreams)) return kChainNotHandled;
  const ColmapLayout l = colmap_layout(cols, num_int, num_fp);
  const uint8_t *cm = static_cast<const uint8_t *>(colmap);
  FusedArgs p{};
  p.qw = static_cast<const uint8_t *>(qw);
  p.s_col = static_cast<const uint16_t *>(s_col);
  p.w_red = static_cast<const uint16_t *>(w_red);
  p.fp_w = static_cast<const uint16_t *>(fp_w);
  p.bias = static_cast<const uint16_t *>(bias);
  p.out = static_cast<uint16_t *>(out);
  p.M = static_cast<int>(rows);
  p.N = static_cast<int>(N);
  p.ldo = static_cast<int>(N);
  p.kbytes = static_cast<int>(bits == 4 ? num_int / 2 : num_int);
  p.F = static_cast<int>(num_fp);
  p.meta_stride = sym ? 1 : 2;
  p.shift = bits == 4 ? 8.0f : 128.0f;
  if (!gemv_ok(p, true)) return kChainNotHandled;
  GemvQuant q{};
  q.x = static_cast<const uint16_t *>(x);
  q.fp_col = reinterpret_cast<const uint16_t *>(cm + l.off_fp);
  q.grp = reinterpret_cast<const uint32_t *>(cm + l.off_grp);
  q.unit = reinterpret_cast<const uint16_t *>(cm + l.off_unit);
  q.gather_unit = reinterpret_cast<const uint16_t *>(cm + l.off_gunit);
  q.gather_cols = reinterpret_cast<const uint16_t *>(cm + l.off_gcols);
  q.cols = static_cast<int>(cols), q.num_int = static_cast<int>(num_int), q.num_fp = static_cast<int>(num_fp);
  q.ngather = static_cast<int>(words[3]);
  q.sym_divisor = sym_divisor;
  if (q.ngather > kGemvWaves * 64) return kChainNotHandled;  // (one gathered unit per thread)
  if (sym) return bits == 4 ? launch_gemv<kInt4, false, kGemvSym>(p, q, st) : launch_gemv<kInt8, false, kGemvSym>(p, q, st);
  if (bits == 4)
    return dtype == QUIK_F16 ? launch_gemv<kInt4, false, kGemvAsym>(p, q, st) : launch_gemv<kInt4, true, kGemvAsym>(p, q, st);
  return dtype == QUIK_F16 ? launch_gemv<kInt8, false, kGemvAsym>(p, q, st) : launch_gemv<kInt8, true, kGemvAsym>(p, q, st);
}

extern "C" int quik_mixed_linear_fwd(const void *qx, const void *qw, const void *meta, const void *s_col,
                                     const void *w_reduced, const void *fp_x, const void *fp_w, const void *bias,
                                     int dtype, int64_t M, int64_t N, int64_t K, int64_t F, int bits, void *out,
                                     void *stream) {
  if (bits != 4 && bits != 8) return QUIK_ERR_BITS;
  if (dtype != QUIK_F16 && dtype != QUIK_BF16) return QUIK_ERR_DTYPE;
  if (F < 0) return QUIK_ERR_SHAPE;
  if (int rc = check_gemm_args(qx, qw, out, M, N, K, bits)) return rc;
  if (M == 0 || N == 0) return QUIK_OK;
  if (!meta || !s_col) return QUIK_ERR_NULL;
  if (F > 0 && (!fp_x || !fp_w)) return QUIK_ERR_NULL;
  if (F % 8 != 0) return QUIK_ERR_ALIGN;
  if (F > 0 && (reinterpret_cast<uintptr_t>(fp_x) % 16 != 0 || reinterpret_cast<uintptr_t>(fp_w) % 16 != 0))
    return QUIK_ERR_ALIGN;
  FusedArgs p;
  p.qx = static_cast<const uint8_t *>(qx);
  p.qw = static_cast<const uint8_t *>(qw);
  p.meta = static_cast<const uint16_t *>(meta);
  p.s_col = static_cast<const uint16_t *>(s_col);
  p.w_red = static_cast<const uint16_t *>(w_reduced);
  p.fp_x = static_cast<const uint16_t *>(fp_x);
  p.fp_w = static_cast<const uint16_t *>(fp_w);
  p.bias = static_cast<const uint16_t *>(bias);
  p.out = static_cast<uint16_t *>(out);
  p.M = static_cast<int>(M);
  p.N = static_cast<int>(N);
  p.ldo = static_cast<int>(N);
  p.kbytes = static_cast<int>(bits == 4 ? K / 2 : K);
  p.F = static_cast<int>(F);
  p.meta_stride = w_reduced ? 2 : 1;
  p.shift = bits == 4 ? 8.0f : 128.0f;
  hipStream_t st = as_stream(stream);
  if (bits == 4) return dtype == QUIK_F16 ? run_fused<kInt4, false>(p, st) : run_fused<kInt4, true>(p, st);
  return dtype == QUIK_F16 ? run_fused<kInt8, false>(p, st) : run_fused<kInt8, true>(p, st);
}

extern "C" int64_t quik_splitk_workspace_bytes(int64_t M, int64_t N, int64_t K, int bits) {
  if (M <= 0 || N <= 0 || K <= 0 || (bits != 4 && bits != 8)) return 0;
  if (bits == 4 ? K % 128 != 0 : K % 64 != 0) return 0;
  return (bits == 4 ? plan_splitk(M, N, K / 64, kSplitMinSteps6, 1, 3) : plan_splitk(M, N, K / 32, kSplitMinSteps8, 1, 2)).bytes;
}

extern "C" int quik_mixed_linear_fwd_fp6(const void *x6, const void *w6, const void *meta, const void *s_col,
                                         const void *w_reduced, const void *bias, int dtype, int64_t M, int64_t N,
                                         int64_t K, int64_t F, void *out, void *stream) {
  return quik_mixed_linear_fwd_fp6_ws(x6, w6, meta, s_col, w_reduced, bias, dtype, M, N, K, F, out, nullptr, 0, stream);
}

extern "C" int quik_mixed_linear_fwd_fp6_ws(const void *x6, const void *w6, const void *meta, const void *s_col,
                                            const void *w_reduced, const void *bias, int dtype, int64_t M, int64_t N,
                                            int64_t K, int64_t F, void *out, void *workspace,
                                            int64_t workspace_bytes, void *stream) {
  if (dtype != QUIK_F16 && dtype != QUIK_BF16) return QUIK_ERR_DTYPE;
  if (M < 0 || N < 0 || K <= 0 || F < 0) return QUIK_ERR_SHAPE;
  if (M == 0 || N == 0) return QUIK_OK;
  if (!x6 || !w6 || !meta || !s_col || !out) return QUIK_ERR_NULL;  // w_reduced == NULL: symmetric activations
  if (K % 128 != 0 || F % 32 != 0) return QUIK_ERR_ALIGN;
  auto misaligned = [](const void *p) { return reinterpret_cast<uintptr_t>(p) % 256 != 0; };
  if (misaligned(x6) || misaligned(w6)) return QUIK_ERR_ALIGN;
  if (M > (1 << 30) || N > (1 << 30) || K > 74496) return QUIK_ERR_RANGE;  // 225 K < 2^24: the fp32 sums stay exact
  Fused6Args p;
  p.xbuf = static_cast<const uint8_t *>(x6);
  p.wbuf = static_cast<const uint8_t *>(w6);
  p.meta = static_cast<const uint16_t *>(meta);
  p.s_col = static_cast<const uint16_t *>(s_col);
  p.w_red = static_cast<const uint16_t *>(w_reduced);
  p.bias = static_cast<const uint16_t *>(bias);
  p.out = static_cast<uint16_t *>(out);
  p.M = static_cast<int>(M);
  p.N = static_cast<int>(N);
  p.ldo = static_cast<int>(N);
  p.K = static_cast<int>(K);
  p.F = static_cast<int>(F);
  p.n_first = 0;
  p.N_total = static_cast<int>(N);
  hipStream_t st = as_stream(stream);
  if (workspace && reinterpret_cast<uintptr_t>(workspace) % 16 != 0) return QUIK_ERR_ALIGN;
  return dtype == QUIK_F16 ? run_fused6<false>(p, st, workspace, workspace_bytes)
                           : run_fused6<true>(p, st, workspace, workspace_bytes);
}

extern "C" int quik_mixed_linear_fwd_tile8(const void *x8, const void *w8, const void *meta, const void *s_col,
                                           const void *w_reduced, const void *bias, int dtype, int64_t M, int64_t N,
                                           int64_t K, int64_t F, void *out, void *stream) {
  return quik_mixed_linear_fwd_tile8_ws(x8, w8, meta, s_col, w_reduced, bias, dtype, M, N, K, F, out, nullptr, 0, stream);
}

extern "C" int quik_mixed_linear_fwd_tile8_ws(const void *x8, const void *w8, const void *meta, const void *s_col,
                                              const void *w_reduced, const void *bias, int dtype, int64_t M, int64_t N,
                                              int64_t K, int64_t F, void *out, void *workspace,
                                              int64_t workspace_bytes, void *stream) {
  if (dtype != QUIK_F16 && dtype != QUIK_BF16) return QUIK_ERR_DTYPE;
  if (M < 0 || N < 0 || K <= 0 || F < 0) return QUIK_ERR_SHAPE;
  if (M == 0 || N == 0) return QUIK_OK;
  if (!x8 || !w8 || !meta || !s_col || !out) return QUIK_ERR_NULL;  // w_reduced == NULL: symmetric activations
  if (K % 64 != 0 || F % 32 != 0) return QUIK_ERR_ALIGN;
  auto misaligned = [](const void *p) { return reinterpret_cast<uintptr_t>(p) % 256 != 0; };
  if (misaligned(x8) || misaligned(w8)) return QUIK_ERR_ALIGN;
  if (M > (1 << 30) || N > (1 << 30) || K > (1 << 24)) return QUIK_ERR_RANGE;
  Fused8Args p;
  p.xbuf = static_cast<const uint8_t *>(x8);
  p.wbuf = static_cast<const uint8_t *>(w8);
  p.meta = static_cast<const uint16_t *>(meta);
  p.s_col = static_cast<const uint16_t *>(s_col);
  p.w_red = static_cast<const uint16_t *>(w_reduced);
  p.bias = static_cast<const uint16_t *>(bias);
  p.out = static_cast<uint16_t *>(out);
  p.M = static_cast<int>(M);
  p.N = static_cast<int>(N);
  p.ldo = static_cast<int>(N);
  p.K = static_cast<int>(K);
  p.F = static_cast<int>(F);
  p.n_first = 0;
  p.N_total = static_cast<int>(N);
  hipStream_t st = as_stream(stream);
  if (workspace && reinterpret_cast<uintptr_t>(workspace) % 16 != 0) return QUIK_ERR_ALIGN;
  return dtype == QUIK_F16 ? run_fused8t<false>(p, st, workspace, workspace_bytes)
                           : run_fused8t<true>(p, st, workspace, workspace_bytes);
}

// ---- the entry point that allocates nothing ------------------------------------------------------------------
// quik_mixed_linear_fwd_tile8_ws with the K-split workspace in a file-scope device array instead of a caller
// buffer: counters (kSplitCounterBytes) followed by the partial accumulators, the size of the largest plan
// plan_splitk makes (tiles x splits <= kMaxCUs workgroups of one 128x128 int32 tile each).  Every GPU that loads this
// library holds its own copy of the array until the process ends.
constexpr int64_t kStaticScratchBytes = kSplitCounterBytes + int64_t(kMaxCUs) * 128 * 128 * 4;
static __device__ __align__(256) uint8_t scratch[kStaticScratchBytes];

namespace quik {
namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
std::atomic<uint8_t *> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device.  In host code the array's name is only a handle for
// hipGetSymbolAddress: the address is looked up once per device, with that device current, and kept.
int scratch_of_current_device(uint8_t **out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    set_last_hip_error(e);
    return QUIK_ERR_LAUNCH;
  }
  if (dev < 0 || dev >= kMaxDevices) return QUIK_ERR_RANGE;
  uint8_t *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    p = g_scratch_ptr[dev].load(std::memory_order_relaxed);
    if (!p) {
      void *sym = nullptr;
      e = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
      if (e != hipSuccess || !sym) {
        set_last_hip_error(e != hipSuccess ? e : hipErrorInvalidSymbol);
        return QUIK_ERR_LAUNCH;
      }
      p = static_cast<uint8_t *>(sym);
      g_scratch_ptr[dev].store(p, std::memory_order_release);
    }
  }
  *out = p;
  return QUIK_OK;
}

// (the counters of `scratch` are cleared with clear_words_kernel in front of each launch that uses them: launches
// leave them at zero, but a launch that failed half way would not, and this array outlives every caller)
}  // namespace
}  // namespace quik

extern "C" int quik_mixed_linear_fwd_tile8_noalloc(const void *x8, const void *w8, const void *meta, const void *s_col,
                                                   const void *w_reduced, const void *bias, int dtype, int64_t M,
                                                   int64_t N, int64_t K, int64_t F, void *out, void *stream) {
  if (dtype != QUIK_F16 && dtype != QUIK_BF16) return QUIK_ERR_DTYPE;
  if (M < 0 || N < 0 || K <= 0 || F < 0) return QUIK_ERR_SHAPE;
  if (K % 64 != 0 || F % 32 != 0) return QUIK_ERR_ALIGN;
  const int64_t need = quik_splitk_workspace_bytes(M, N, K, 8);
  if (need > kStaticScratchBytes) return QUIK_ERR_RANGE;  // a K split larger than the static array holds
  if (need == 0 || M == 0 || N == 0)                      // no K split for this shape: no scratch memory involved
    return quik_mixed_linear_fwd_tile8_ws(x8, w8, meta, s_col, w_reduced, bias, dtype, M, N, K, F, out, nullptr, 0, stream);
  if (!x8 || !w8 || !meta || !s_col || !out) return QUIK_ERR_NULL;
  uint8_t *ws = nullptr;
  if (int rc = scratch_of_current_device(&ws)) return rc;
  hipLaunchKernelGGL(clear_words_kernel, dim3(static_cast<unsigned>(kSplitCounterBytes / 4 / 256)), dim3(256), 0,
                     as_stream(stream), reinterpret_cast<uint32_t *>(ws), static_cast<int>(kSplitCounterBytes / 4));
  if (int rc = check_launch()) return rc;
  return quik_mixed_linear_fwd_tile8_ws(x8, w8, meta, s_col, w_reduced, bias, dtype, M, N, K, F, out, ws,
                                        kStaticScratchBytes, stream);
}
