// Integer GEMMs of the MixedQLinear forward path on CDNA4 (gfx950) matrix cores:
//   int4 x int4 -> int32, int8 x int8 -> int32 (the unfused ops), and the fused forward
//   out = dtype( f32(acc) * (s_row * s_col) + (zero + 2^(bits-1) s_row) * w_red + fp_x fp_w^T + bias ).
//
// Operands are "TN": A [M, K] and B [N, K] are both K-contiguous, which is the native operand
// order of v_mfma_i32_32x32x32_i8 (lane l supplies 16 consecutive K bytes of row l%32, K half
// l/32).  Because A and B fragments are fetched with the same lane->K mapping, any permutation
// of K inside one instruction is harmless; the int4 path exploits that:
//   a packed dword w holds nibbles n0..n7;  lo = (w << 4) & 0xF0F0F0F0 is int8x4 {16 n0, 16 n2,
//   16 n4, 16 n6},  hi = w & 0xF0F0F0F0 is {16 n1, 16 n3, 16 n5, 16 n7}.  Both operands are
//   unpacked the same way, products come out 256x too large, and the exact accumulator is
//   recovered with an arithmetic shift by 8 (needs 16384 K < 2^31, i.e. K < 131072).
// There is no int4 MFMA on CDNA4; int4 saves HBM/LDS bytes only.
//
// Structure: one workgroup computes a BM x BN tile with WAVES_M x WAVES_N wavefronts, each wave
// a (BM/WAVES_M) x (BN/WAVES_N) sub-tile of 32x32 MFMA blocks held in registers.  K is streamed
// in stages of BKB bytes per row through a double-buffered LDS tile (global -> registers ->
// LDS, next stage prefetched while the current one feeds the MFMAs); LDS rows are padded by 16
// bytes so the 16-byte fragment reads of 32 consecutive rows fall in distinct banks.  The fused
// kernel reuses the same pipeline for the fp16/bf16 outlier GEMM (v_mfma_f32_32x32x16_f16 /
// _bf16) after the integer accumulators have been converted to fp32 in place, so the outliers
// cost extra K iterations and no extra registers.  Workgroup ids are remapped so that the ids
// that land on one XCD (id % 8) cover neighbouring tiles and share their L2.
#include "common.h"

namespace quik {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

enum Mode { kInt4 = 0, kInt8 = 1, kF16 = 2, kBF16 = 3 };

template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, int BKB_>
struct Cfg {
  static constexpr int BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, BKB = BKB_;
  static constexpr int kThreads = WAVES_M * WAVES_N * 64;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int MI = WM / 32, NI = WN / 32;
  static constexpr int LDS_STRIDE = BKB + 16;
  static constexpr int A_BYTES = BM * LDS_STRIDE, B_BYTES = BN * LDS_STRIDE;
  static constexpr int STAGE = A_BYTES + B_BYTES;
  static constexpr int SMEM = 2 * STAGE;
  static constexpr int CHUNKS = BKB / 16;  // 16-byte chunks per tile row
  static constexpr int A_LOADS = (BM * CHUNKS + kThreads - 1) / kThreads;
  static constexpr int B_LOADS = (BN * CHUNKS + kThreads - 1) / kThreads;
  static_assert(WM % 32 == 0 && WN % 32 == 0 && BKB % 32 == 0, "tile shape");
};

// One operand stream: global rows -> registers -> LDS.
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

__device__ __forceinline__ void unpack_i4(const v4i w, v4i &f0, v4i &f1) {
  constexpr int kMask = static_cast<int>(0xF0F0F0F0u);
  f0 = v4i{(w.x << 4) & kMask, w.x & kMask, (w.y << 4) & kMask, w.y & kMask};
  f1 = v4i{(w.z << 4) & kMask, w.z & kMask, (w.w << 4) & kMask, w.w & kMask};
}

// Accumulates A_tile x B_tile^T over `kbytes` bytes of K into acc (int32 or fp32 by MODE).
template <class C, int MODE, typename AccT>
__device__ __forceinline__ void mainloop(const uint8_t *__restrict__ A, int64_t lda, int rows_a,
                                         const uint8_t *__restrict__ B, int64_t ldb, int rows_b, int kbytes,
                                         uint8_t *smem, AccT (&acc)[C::MI][C::NI]) {
  OperandLoader<C::BM, C::A_LOADS, C> la;
  OperandLoader<C::BN, C::B_LOADS, C> lb;
  la.init(A, lda, rows_a, 0);
  lb.init(B, ldb, rows_b, C::A_BYTES);

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;
  const int a_frag = (wm * C::WM + (lane & 31)) * C::LDS_STRIDE + (lane >> 5) * 16;
  const int b_frag = C::A_BYTES + (wn * C::WN + (lane & 31)) * C::LDS_STRIDE + (lane >> 5) * 16;

  const int stages = (kbytes + C::BKB - 1) / C::BKB;
  la.fetch(0, kbytes);
  lb.fetch(0, kbytes);
  la.stash(smem, 0);
  lb.stash(smem, 0);
  __syncthreads();

  for (int kt = 0; kt < stages; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < stages) {
      la.fetch((kt + 1) * C::BKB, kbytes);
      lb.fetch((kt + 1) * C::BKB, kbytes);
    }
    const uint8_t *sa = smem + cur * C::STAGE + a_frag;
    const uint8_t *sb = smem + cur * C::STAGE + b_frag;
#pragma unroll
    for (int ks = 0; ks < C::BKB / 32; ++ks) {
      v4i ra[C::MI];
#pragma unroll
      for (int mi = 0; mi < C::MI; ++mi)
        ra[mi] = *reinterpret_cast<const v4i *>(sa + mi * 32 * C::LDS_STRIDE + ks * 32);
      if constexpr (MODE == kInt4) {
        v4i a0[C::MI], a1[C::MI];
#pragma unroll
        for (int mi = 0; mi < C::MI; ++mi) unpack_i4(ra[mi], a0[mi], a1[mi]);
#pragma unroll
        for (int ni = 0; ni < C::NI; ++ni) {
          const v4i rb = *reinterpret_cast<const v4i *>(sb + ni * 32 * C::LDS_STRIDE + ks * 32);
          v4i b0, b1;
          unpack_i4(rb, b0, b1);
#pragma unroll
          for (int mi = 0; mi < C::MI; ++mi) {
            acc[mi][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0[mi], b0, acc[mi][ni], 0, 0, 0);
            acc[mi][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1[mi], b1, acc[mi][ni], 0, 0, 0);
          }
        }
      } else {
#pragma unroll
        for (int ni = 0; ni < C::NI; ++ni) {
          const v4i rb = *reinterpret_cast<const v4i *>(sb + ni * 32 * C::LDS_STRIDE + ks * 32);
#pragma unroll
          for (int mi = 0; mi < C::MI; ++mi) {
            if constexpr (MODE == kInt8) {
              acc[mi][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ra[mi], rb, acc[mi][ni], 0, 0, 0);
            } else if constexpr (MODE == kF16) {
              acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, ra[mi]),
                                                                   __builtin_bit_cast(v8h, rb), acc[mi][ni], 0, 0, 0);
            } else {
              acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, ra[mi]),
                                                                    __builtin_bit_cast(v8bf, rb), acc[mi][ni], 0, 0, 0);
            }
          }
        }
      }
    }
    if (kt + 1 < stages) {
      la.stash(smem, cur ^ 1);
      lb.stash(smem, cur ^ 1);
    }
    __syncthreads();
  }
}

// Workgroup id -> tile.  Hardware deals consecutive workgroup ids round-robin to the 8 XCDs;
// ids congruent mod 8 therefore share an L2.  Give each XCD a contiguous run of tiles, with M
// fastest, so concurrently resident tiles of an XCD share B rows and cover all of A.
__device__ __forceinline__ bool tile_of_block(int tiles_m, int tiles_n, int &tm, int &tn) {
  const int total = tiles_m * tiles_n;
  const int per_xcd = (total + 7) / 8;
  const int logical = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (logical >= total) return false;
  tm = logical % tiles_m;
  tn = logical / tiles_m;
  return true;
}

// Row/column of accumulator register v of a 32x32 block for this lane:
//   column = lane % 32, row = 8 * (v / 4) + 4 * (lane / 32) + v % 4.
__device__ __forceinline__ int acc_row(int v, int lane) { return 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3); }

template <class C, int MODE>
__global__ __launch_bounds__(C::kThreads) void gemm_i32_kernel(const uint8_t *__restrict__ A,
                                                               const uint8_t *__restrict__ B, int32_t *__restrict__ Cm,
                                                               int M, int N, int kbytes, int tiles_m, int tiles_n) {
  extern __shared__ __align__(16) uint8_t smem[];
  int tm, tn;
  if (!tile_of_block(tiles_m, tiles_n, tm, tn)) return;
  const int m0 = tm * C::BM, n0 = tn * C::BN;
  v16i acc[C::MI][C::NI];
#pragma unroll
  for (int mi = 0; mi < C::MI; ++mi)
#pragma unroll
    for (int ni = 0; ni < C::NI; ++ni)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0;
  mainloop<C, MODE>(A + int64_t(m0) * kbytes, kbytes, M - m0, B + int64_t(n0) * kbytes, kbytes, N - n0, kbytes, smem,
                    acc);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;
  constexpr int kShift = MODE == kInt4 ? 8 : 0;
#pragma unroll
  for (int mi = 0; mi < C::MI; ++mi)
#pragma unroll
    for (int ni = 0; ni < C::NI; ++ni) {
      const int n = n0 + wn * C::WN + ni * 32 + (lane & 31);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + wm * C::WM + mi * 32 + acc_row(v, lane);
        if (m < M && n < N) Cm[int64_t(m) * N + n] = acc[mi][ni][v] >> kShift;
      }
    }
}

struct FusedArgs {
  const uint8_t *qx, *qw;
  const uint16_t *meta, *s_col, *w_red, *fp_x, *fp_w, *bias;
  uint16_t *out;
  int M, N, kbytes, F;
  int meta_stride;  // 2: (scale, zero) pairs; 1: scales only (symmetric)
  float shift;
};

template <class C, int MODE, bool BF16>
__global__ __launch_bounds__(C::kThreads) void gemm_fused_kernel(FusedArgs p, int tiles_m, int tiles_n) {
  extern __shared__ __align__(16) uint8_t smem[];
  int tm, tn;
  if (!tile_of_block(tiles_m, tiles_n, tm, tn)) return;
  const int m0 = tm * C::BM, n0 = tn * C::BN;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;
  constexpr int kShift = MODE == kInt4 ? 8 : 0;

  v16f accf[C::MI][C::NI];
  {
    v16i acc[C::MI][C::NI];
#pragma unroll
    for (int mi = 0; mi < C::MI; ++mi)
#pragma unroll
      for (int ni = 0; ni < C::NI; ++ni)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0;
    mainloop<C, MODE>(p.qx + int64_t(m0) * p.kbytes, p.kbytes, p.M - m0, p.qw + int64_t(n0) * p.kbytes, p.kbytes,
                      p.N - n0, p.kbytes, smem, acc);
    // acc -> f32(acc) * (s_row * s_col), in place
    float sc[C::NI];
#pragma unroll
    for (int ni = 0; ni < C::NI; ++ni) {
      const int n = n0 + wn * C::WN + ni * 32 + (lane & 31);
      sc[ni] = to_f32<BF16>(p.s_col[n < p.N ? n : p.N - 1]);
    }
#pragma unroll
    for (int mi = 0; mi < C::MI; ++mi)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + wm * C::WM + mi * 32 + acc_row(v, lane);
        const float s = to_f32<BF16>(p.meta[int64_t(m < p.M ? m : p.M - 1) * p.meta_stride]);
#pragma unroll
        for (int ni = 0; ni < C::NI; ++ni)
          accf[mi][ni][v] = static_cast<float>(acc[mi][ni][v] >> kShift) * (s * sc[ni]);
      }
  }
  if (p.F > 0) {
    mainloop<C, BF16 ? kBF16 : kF16>(reinterpret_cast<const uint8_t *>(p.fp_x) + int64_t(m0) * p.F * 2,
                                     int64_t(p.F) * 2, p.M - m0,
                                     reinterpret_cast<const uint8_t *>(p.fp_w) + int64_t(n0) * p.F * 2,
                                     int64_t(p.F) * 2, p.N - n0, p.F * 2, smem, accf);
  }
  float wr[C::NI], bs[C::NI];
#pragma unroll
  for (int ni = 0; ni < C::NI; ++ni) {
    const int n = n0 + wn * C::WN + ni * 32 + (lane & 31);
    const int nc = n < p.N ? n : p.N - 1;
    wr[ni] = p.w_red ? to_f32<BF16>(p.w_red[nc]) : 0.0f;
    bs[ni] = p.bias ? to_f32<BF16>(p.bias[nc]) : 0.0f;
  }
#pragma unroll
  for (int mi = 0; mi < C::MI; ++mi)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int m = m0 + wm * C::WM + mi * 32 + acc_row(v, lane);
      float zs = 0.0f;
      if (p.w_red) {
        const int64_t mc = m < p.M ? m : p.M - 1;
        const float s = to_f32<BF16>(p.meta[2 * mc]);
        const float z = to_f32<BF16>(p.meta[2 * mc + 1]);
        zs = z + p.shift * s;
      }
#pragma unroll
      for (int ni = 0; ni < C::NI; ++ni) {
        const int n = n0 + wn * C::WN + ni * 32 + (lane & 31);
        const float t = accf[mi][ni][v] + (zs * wr[ni] + bs[ni]);
        if (m < p.M && n < p.N) p.out[int64_t(m) * p.N + n] = from_f32<BF16>(t);
      }
    }
}

using CfgL = Cfg<256, 256, 2, 2, 64>;  // prefill: 128x128 per wave, 256 accumulator registers
using CfgM = Cfg<128, 128, 2, 2, 64>;  // mid-size M or few tiles
using CfgS = Cfg<32, 128, 1, 4, 64>;   // decode: M <= 32

template <class C>
int pick_grid(int64_t M, int64_t N, int &tiles_m, int &tiles_n) {
  tiles_m = static_cast<int>((M + C::BM - 1) / C::BM);
  tiles_n = static_cast<int>((N + C::BN - 1) / C::BN);
  const int64_t total = int64_t(tiles_m) * tiles_n;
  return static_cast<int>(((total + 7) / 8) * 8);
}

template <typename K>
int prepare(K kern, int smem) {
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) {
      set_last_hip_error(e);
      return QUIK_ERR_LAUNCH;
    }
  }
  return QUIK_OK;
}

template <class C, int MODE>
int launch_i32(const uint8_t *A, const uint8_t *B, int32_t *Cm, int64_t M, int64_t N, int64_t kbytes,
               hipStream_t st) {
  int tiles_m, tiles_n;
  const int grid = pick_grid<C>(M, N, tiles_m, tiles_n);
  auto kern = gemm_i32_kernel<C, MODE>;
  if (int rc = prepare(kern, C::SMEM)) return rc;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(C::kThreads), C::SMEM, st, A, B, Cm, static_cast<int>(M),
                     static_cast<int>(N), static_cast<int>(kbytes), tiles_m, tiles_n);
  return check_launch();
}

template <class C, int MODE, bool BF16>
int launch_fused(const FusedArgs &p, hipStream_t st) {
  int tiles_m, tiles_n;
  const int grid = pick_grid<C>(p.M, p.N, tiles_m, tiles_n);
  auto kern = gemm_fused_kernel<C, MODE, BF16>;
  if (int rc = prepare(kern, C::SMEM)) return rc;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(C::kThreads), C::SMEM, st, p, tiles_m, tiles_n);
  return check_launch();
}

// 0: large tile, 1: medium, 2: small
int pick_cfg(int64_t M, int64_t N) {
  if (M <= 32) return 2;
  const int64_t big_tiles = ((M + 255) / 256) * ((N + 255) / 256);
  if (M <= 128 || big_tiles < 128) return 1;
  return 0;
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

}  // namespace
}  // namespace quik

using namespace quik;

extern "C" int quik_int4_matmul(const uint8_t *A, const uint8_t *B, int32_t *C, int64_t M, int64_t N, int64_t K,
                                void *stream) {
  if (int rc = check_gemm_args(A, B, C, M, N, K, 4)) return rc;
  if (M == 0 || N == 0) return QUIK_OK;
  hipStream_t st = as_stream(stream);
  switch (pick_cfg(M, N)) {
    case 0: return launch_i32<CfgL, kInt4>(A, B, C, M, N, K / 2, st);
    case 1: return launch_i32<CfgM, kInt4>(A, B, C, M, N, K / 2, st);
    default: return launch_i32<CfgS, kInt4>(A, B, C, M, N, K / 2, st);
  }
}

extern "C" int quik_int8_matmul(const int8_t *A, const int8_t *B, int32_t *C, int64_t M, int64_t N, int64_t K,
                                void *stream) {
  if (int rc = check_gemm_args(A, B, C, M, N, K, 8)) return rc;
  if (M == 0 || N == 0) return QUIK_OK;
  hipStream_t st = as_stream(stream);
  const uint8_t *a = reinterpret_cast<const uint8_t *>(A), *b = reinterpret_cast<const uint8_t *>(B);
  switch (pick_cfg(M, N)) {
    case 0: return launch_i32<CfgL, kInt8>(a, b, C, M, N, K, st);
    case 1: return launch_i32<CfgM, kInt8>(a, b, C, M, N, K, st);
    default: return launch_i32<CfgS, kInt8>(a, b, C, M, N, K, st);
  }
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
  p.kbytes = static_cast<int>(bits == 4 ? K / 2 : K);
  p.F = static_cast<int>(F);
  p.meta_stride = w_reduced ? 2 : 1;
  p.shift = bits == 4 ? 8.0f : 128.0f;
  hipStream_t st = as_stream(stream);
  const int cfg = pick_cfg(M, N);
#define QUIK_FUSED(CFG)                                                                                     \
  if (bits == 4)                                                                                            \
    return dtype == QUIK_F16 ? launch_fused<CFG, kInt4, false>(p, st) : launch_fused<CFG, kInt4, true>(p, st); \
  else                                                                                                      \
    return dtype == QUIK_F16 ? launch_fused<CFG, kInt8, false>(p, st) : launch_fused<CFG, kInt8, true>(p, st);
  if (cfg == 0) {
    QUIK_FUSED(CfgL)
  } else if (cfg == 1) {
    QUIK_FUSED(CfgM)
  } else {
    QUIK_FUSED(CfgS)
  }
#undef QUIK_FUSED
}
