// Skinny GEMM for at most 32 token rows (decode): the weights are read exactly once, straight from
// global memory into MFMA operand registers, and the problem is bound by that stream.
//
// A slab is 32 output columns (one MFMA row block) times all token rows.  A workgroup of WAVES
// wavefronts walks over slabs blockIdx.x, blockIdx.x + gridDim.x, ...; inside a slab K is cut into
// 128-byte chunks per row and wave w takes chunks w, w + WAVES, ...  Every wave runs one
// continuous stream of (slab, chunk) items with NB register sets in rotation, so NB - 1 chunks
// are always in flight ahead of the one being multiplied, across slab boundaries too: the memory
// latency is paid once per wave, not once per slab.
// The MFMA wants lane l to hold 16 bytes of weight row l % 32 at K half l / 32 of a 32-byte step.  Loading them
// that way asks for 32 bytes of 32 different rows per instruction, and the memory path then delivers 13-24 % less
// than when an instruction covers whole 128-byte lines (measured with the loads rearranged and the results
// ignored).  So load i of a chunk has lane l fetch 16-byte piece l % 8 of row 8 i + l / 8 (eight whole lines), and
// at multiply time the wave passes the chunk through 4 KB of LDS of its own, written as a row-major 32 x 128 byte
// tile (pieces XOR-swizzled by (row / 2) % 8, so that the writes and the reads below are conflict-free) and read
// back in the operand layout.  The LDS of a wave executes in order: no waits beyond the data dependences.
// The token rows take the same route in the fused form (rows past M repeat the last one), are loaded in the operand
// layout directly in the plain integer form, or are read from their LDS copy (XLDS); int4: the same in-register
// nibble split as the large tiles.  The fp16/bf16 outlier columns are split over the waves the same way; those loads and
// the epilogue's per-row / per-column scalars are requested when a slab starts.  At the end of a
// slab the waves' partial accumulators (int32, exact in any order; fp32 outlier sums, added in
// wave order) meet in LDS, and every wave finalises 16 / WAVES of the 16 values a lane owns with
// the same epilogue formula as the large tiles.
//
// XLDS: the token operand lives in LDS.  Without it every slab re-reads all token rows from L2, as many bytes
// as the slab's weights when there are 32 rows, and that traffic, not the weight stream, sets the time (a
// 28672 x 7936 int4 layer: 34 us with one token row, 57 us with 32).  When the rows fit (rows x K bytes beside
// the reduction area), each persistent workgroup copies them once, in the order the lanes read them
// ([chunk][step][K half][row], 16 bytes each: conflict-free), and only the weights are streamed.
#pragma once
#include "gemm_kernels.h"

namespace quik {

constexpr int kDecodeChunk = 128;  // K bytes per row and wave turn
constexpr int kDecodeSteps = kDecodeChunk / 32;

// reduction area: int32 partial sums and, for the fused form, fp32 outlier sums; with XLDS the two share one
// area (one after the other) to leave room for the token rows
// behind it, in the fused form: 2 KB in which a slab's 32 x 32 outputs are gathered into whole row segments
constexpr int kDecodeStage = 2048;
template <int WAVES, bool FUSED, bool XLDS = false>
constexpr int decode_smem() {
  return WAVES * 4096 * (FUSED && !XLDS ? 2 : 1) + (FUSED ? kDecodeStage : 0);
}
// bytes of the LDS copy of `rows` token rows of `kbytes` bytes (whole 1 KB copies)
inline int64_t decode_x_lds_bytes(int64_t rows, int64_t kbytes) {
  const int64_t units = (kbytes + kDecodeChunk - 1) / kDecodeChunk * kDecodeSteps * 2 * rows;
  return (units + 63) / 64 * 1024;
}

// FUSED: p.out receives the MixedQLinear output.  !FUSED: Cm receives the int32 product.
template <int MODE, bool BF16, bool FUSED, int WAVES, bool XLDS = false>
__global__ __launch_bounds__(WAVES * 64) void gemm_decode_kernel(FusedArgs args, int32_t *__restrict__ Cm, int ldc) {
  static_assert(WAVES == 4 || WAVES == 8, "16 values per lane are split over the waves");
  // plain locals: the lambdas below capture by reference, and a captured argument struct ends up in scratch
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
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 31, h = lane >> 5;
  const int mrow = r < p.M ? r : p.M - 1;  // rows past the edge are computed on valid memory, never stored
  const int kbytes = p.kbytes;
  const int nchunks = (kbytes + kDecodeChunk - 1) / kDecodeChunk;
  const int slabs = (p.N + 31) / 32;
  const int stride = gridDim.x;
  const uint8_t *xp = p.qx + int64_t(mrow) * kbytes + h * 16;
  constexpr int VPW = 16 / WAVES;                             // values per lane this wave finalises
  constexpr int kFpEarly = FUSED ? 2 : 0;                     // outlier pieces requested at slab start
  using FpOps = FragOps<BF16 ? kBF16 : kF16>;

  // Every load below is issued unconditionally, from a clamped (valid) address, and what must read as zero is
  // masked when it is used: with loads under a branch the number of loads in flight is unknown at compile time
  // and every wait becomes a wait for all of them, which empties the prefetch queue before each chunk.
  struct Buf {
    v4i w[kDecodeSteps], x[XLDS ? 1 : kDecodeSteps];
    int keep;  // all ones: this lane's piece of the chunk exists; zero: empty item or past the row's end
  };
  // ---- XLDS: copy the token rows into LDS, 16-byte unit u = ((chunk step) * 2 + K half) * M + row
  const uint8_t *x_lds = smem + decode_smem<WAVES, FUSED, XLDS>();
  auto copy_token_rows = [&]() __attribute__((always_inline)) {
    const int units = nchunks * kDecodeSteps * 2 * p.M;
    const uint32_t lds_base = lds_address(smem + decode_smem<WAVES, FUSED, XLDS>());
    for (int u0 = __builtin_amdgcn_readfirstlane(wave) * 64; u0 < units; u0 += WAVES * 64) {
      const int u = u0 + lane < units ? u0 + lane : units - 1;  // the last copy is padded with a valid unit
      const int cs = u / (2 * p.M), rem = u - cs * 2 * p.M;
      const int hh = rem >= p.M ? 1 : 0, row = rem - hh * p.M;
      int off = cs * 32 + hh * 16;
      off = off < kbytes ? off : 0;  // past the row's end: the weights of these positions are zeroed below
      dma_load16(p.qx, static_cast<uint32_t>(row * kbytes + off), lds_base + u0 * 16);
    }
  };
  if constexpr (XLDS) x_lds += (h * p.M + mrow) * 16;  // this lane's unit inside a step
  const int x_step = 2 * p.M * 16;
  // ---- loader: item (ld_slab, ld_c) -> b, then advance to this wave's next item
  int ld_slab = blockIdx.x, ld_c = wave;
  auto issue = [&](Buf &b) __attribute__((always_inline)) {
    const bool live = ld_slab < slabs && ld_c < nchunks;
    const int base = ld_c * kDecodeChunk;
    const int piece = base + (lane & 7) * 16;     // this lane's 16 bytes of the chunk's 128
    const bool ok = live && piece < kbytes;
    b.keep = ok ? -1 : 0;
    const int piece_c = ok ? piece : 0;
    const int slab_c = ld_slab < slabs ? ld_slab : slabs - 1;
#pragma unroll
    for (int s = 0; s < kDecodeSteps; ++s) {
      const int n = slab_c * 32 + 8 * s + (lane >> 3);
      b.w[s] = *reinterpret_cast<const v4i *>(p.qw + int64_t(n < p.N ? n : p.N - 1) * kbytes + piece_c);
      if constexpr (!XLDS) {
        if constexpr (FUSED) {  // whole lines as well (the fused form has a second 4 KB per wave to pass them through)
          const int m = 8 * s + (lane >> 3);
          b.x[s] = *reinterpret_cast<const v4i *>(p.qx + int64_t(m < p.M ? m : p.M - 1) * kbytes + piece_c);
        } else {  // (zero weights stand against whatever is read in place of a missing piece)
          const int off = base + s * 32;
          b.x[s] = *reinterpret_cast<const v4i *>(xp + (live && off + h * 16 < kbytes ? off : -h * 16));
        }
      }
    }
    ld_c += WAVES;
    if (ld_c >= nchunks) {  // every wave has at least one (possibly empty) item per slab
      ld_c = wave;
      ld_slab += stride;
    }
  };

  // ---- per-slab state requested when the slab starts: outlier pieces and epilogue scalars
  const int fbytes = FUSED ? p.F * 2 : 0;
  v4i fwe[kFpEarly > 0 ? kFpEarly : 1], fxe[kFpEarly > 0 ? kFpEarly : 1];
  float srow = 0.0f, zs = 0.0f;
  uint16_t e_sc[VPW], e_wr[VPW], e_bs[VPW];  // raw: converted where they are used, so that nothing waits here
  const uint16_t *wr_ptr = p.w_red ? p.w_red : p.s_col, *bs_ptr = p.bias ? p.bias : p.s_col;
  const uint8_t *fx = nullptr;
  if constexpr (FUSED) {
    fx = reinterpret_cast<const uint8_t *>(p.fp_x) + int64_t(mrow) * fbytes + h * 16;
    srow = to_f32<BF16>(p.meta[int64_t(mrow) * p.meta_stride]);
    zs = p.w_red ? to_f32<BF16>(p.meta[2 * int64_t(mrow) + 1]) + p.shift * srow : 0.0f;
    if constexpr (MODE == kInt4) srow *= 0.00390625f;  // the int4 accumulators carry a factor 256
  }
  // this wave's outlier pieces of the token rows are the same for every slab: loaded once
  if constexpr (FUSED) {
    if (fbytes > 0) {
#pragma unroll
      for (int i = 0; i < kFpEarly; ++i) {
        const int off = (wave + i * WAVES) * 32;
        fxe[i] = *reinterpret_cast<const v4i *>(fx + (off + h * 16 < fbytes ? off : -h * 16));
      }
    }
  }
  auto fp_row = [&](int slab) __attribute__((always_inline)) {
    const int n = slab * 32 + r;
    return reinterpret_cast<const uint8_t *>(p.fp_w) + int64_t(n < p.N ? n : p.N - 1) * fbytes + h * 16;
  };
  auto slab_begin = [&](int slab) __attribute__((always_inline)) {
    if constexpr (FUSED) {
      if (slab >= slabs) return;
      if (fbytes > 0) {  // (uniform over the launch)
        const uint8_t *fw = fp_row(slab);
#pragma unroll
        for (int i = 0; i < kFpEarly; ++i) {
          const int off = (wave + i * WAVES) * 32;
          const int off_c = off + h * 16 < fbytes ? off : -h * 16;  // a missing piece reads the row's start, masked in slab_end
          fwe[i] = *reinterpret_cast<const v4i *>(fw + off_c);
        }
      }
#pragma unroll
      for (int j = 0; j < VPW; ++j) {
        const int v = wave * VPW + j;
        const int n = slab * 32 + 8 * (v >> 2) + 4 * h + (v & 3);  // accumulator register v of this lane: see acc_col()
        const int nn = n < p.N ? n : p.N - 1;
        e_sc[j] = p.s_col[nn];
        e_wr[j] = wr_ptr[nn];
        e_bs[j] = bs_ptr[nn];
      }
    }
  };

  v16i acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0;
  auto multiply = [&](const Buf &b, int chunk) __attribute__((always_inline)) {
    const uint8_t *xs = x_lds + (chunk < nchunks ? chunk : 0) * kDecodeSteps * x_step;  // (empty items: zero weights)
    uint8_t *tile = smem + wave * 4096;  // this wave's corner of the reduction area, idle between slab ends
    constexpr bool kXTile = FUSED && !XLDS;
    uint8_t *xtile = smem + (WAVES + wave) * 4096;  // (the fp32 half of the reduction area)
#pragma unroll
    for (int s = 0; s < kDecodeSteps; ++s) {
      const int at = s * 1024 + (lane >> 3) * 128 + (((lane & 7) ^ ((4 * s + (lane >> 4)) & 7)) << 4);
      *reinterpret_cast<v4i *>(tile + at) = v4i{b.w[s].x & b.keep, b.w[s].y & b.keep, b.w[s].z & b.keep, b.w[s].w & b.keep};
      if constexpr (kXTile) *reinterpret_cast<v4i *>(xtile + at) = b.x[s];
    }
#pragma unroll
    for (int s = 0; s < kDecodeSteps; ++s) {
      v4i wu[FragOps<MODE>::H], xu[FragOps<MODE>::H];
      FragOps<MODE>::unpack(*reinterpret_cast<const v4i *>(tile + r * 128 + (((2 * s + h) ^ ((r >> 1) & 7)) << 4)), wu);
      if constexpr (XLDS) {
        FragOps<MODE>::unpack(*reinterpret_cast<const v4i *>(xs + s * x_step), xu);
      } else if constexpr (kXTile) {
        FragOps<MODE>::unpack(*reinterpret_cast<const v4i *>(xtile + r * 128 + (((2 * s + h) ^ ((r >> 1) & 7)) << 4)), xu);
      } else {
        FragOps<MODE>::unpack(b.x[s], xu);
      }
#pragma unroll
      for (int k = 0; k < FragOps<MODE>::H; ++k) FragOps<MODE>::mma(xu[k], wu[k], acc);
    }
  };

  int32_t *red_i = reinterpret_cast<int32_t *>(smem);
  constexpr bool kTwoPhase = XLDS && FUSED;  // fp32 sums go through the int32 area after it has been read
  float *red_f = reinterpret_cast<float *>(smem + (kTwoPhase ? 0 : WAVES * 4096));
  // ---- end of a slab: outlier product, cross-wave reduction, epilogue, stores
  auto slab_end = [&](int slab) __attribute__((always_inline)) {
    v16f accf;
#pragma unroll
    for (int v = 0; v < 16; ++v) accf[v] = 0.0f;
    if constexpr (FUSED) {
#pragma unroll
      for (int i = 0; i < kFpEarly; ++i) {
        const int keep = fbytes > 0 && (wave + i * WAVES) * 32 + h * 16 < fbytes ? -1 : 0;
        if (fbytes > 0)
          FpOps::mma(fxe[i], v4i{fwe[i].x & keep, fwe[i].y & keep, fwe[i].z & keep, fwe[i].w & keep}, accf);
      }
      const uint8_t *fw = fp_row(slab);
      for (int off = (wave + kFpEarly * WAVES) * 32; off < fbytes; off += WAVES * 32) {
        v4i wv = v4i{0, 0, 0, 0}, xv = v4i{0, 0, 0, 0};
        if (off + h * 16 < fbytes) {
          wv = *reinterpret_cast<const v4i *>(fw + off);
          xv = *reinterpret_cast<const v4i *>(fx + off);
        }
        FpOps::mma(xv, wv, accf);
      }
    }
    // partial sums -> LDS, layout [wave][value][lane]: consecutive lanes, consecutive words
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      red_i[(wave * 16 + v) * 64 + lane] = acc[v];
      if constexpr (FUSED && !kTwoPhase) red_f[(wave * 16 + v) * 64 + lane] = accf[v];
      acc[v] = 0;
    }
    __syncthreads();
    // wave w finalises values [w * VPW, (w + 1) * VPW) of every lane
    int32_t tis[VPW];
    float tfs[VPW];
#pragma unroll
    for (int j = 0; j < VPW; ++j) {
      const int v = wave * VPW + j;
      tis[j] = 0;
      tfs[j] = 0.0f;
#pragma unroll
      for (int q = 0; q < WAVES; ++q) {
        tis[j] += red_i[(q * 16 + v) * 64 + lane];
        if constexpr (FUSED && !kTwoPhase) tfs[j] += red_f[(q * 16 + v) * 64 + lane];
      }
    }
    if constexpr (kTwoPhase) {
      __syncthreads();
#pragma unroll
      for (int v = 0; v < 16; ++v) red_f[(wave * 16 + v) * 64 + lane] = accf[v];
      __syncthreads();
#pragma unroll
      for (int j = 0; j < VPW; ++j) {
#pragma unroll
        for (int q = 0; q < WAVES; ++q) tfs[j] += red_f[(q * 16 + wave * VPW + j) * 64 + lane];
      }
    }
    // Fused form: a lane holds single values of 2-byte outputs, one row each: stored as they are, every store
    // instruction would touch 32 lines for 128 bytes.  They are gathered in LDS and leave as 16-byte pieces of
    // row segments (when the output's alignment allows it).
    uint16_t *stage = reinterpret_cast<uint16_t *>(smem + decode_smem<WAVES, FUSED, XLDS>() - kDecodeStage);
    const bool staged = FUSED && (p.ldo & 7) == 0 && (reinterpret_cast<uintptr_t>(p.out) & 15) == 0;
#pragma unroll
    for (int j = 0; j < VPW; ++j) {
      const int v = wave * VPW + j;
      const int32_t ti = tis[j];
      const float tf = tfs[j];
      const int nl = 8 * (v >> 2) + 4 * h + (v & 3), n = slab * 32 + nl;
      if constexpr (FUSED) {
        const float sc = to_f32<BF16>(e_sc[j]);
        const float wr = p.w_red ? to_f32<BF16>(e_wr[j]) : 0.0f, bs = p.bias ? to_f32<BF16>(e_bs[j]) : 0.0f;
        const float val = (static_cast<float>(ti) * (srow * sc) + tf) + (zs * wr + bs);
        if (staged) {
          stage[r * 32 + nl] = from_f32<BF16>(val);
        } else if (r < p.M && n < p.N) {
          p.out[int64_t(r) * p.ldo + n] = from_f32<BF16>(val);
        }
      } else {
        if (r < p.M && n < p.N) Cm[int64_t(r) * ldc + n] = MODE == kInt4 ? (ti >> 8) : ti;
      }
    }
    __syncthreads();  // the next slab's partial sums reuse the area
    if constexpr (FUSED) {
      // (the staging area is written again only behind the next slab's barriers)
      if (staged && threadIdx.x < 128) {
        const int row = threadIdx.x >> 2, n0 = slab * 32 + (threadIdx.x & 3) * 8;
        if (row < p.M && n0 < p.N) {
          const v4i d = *reinterpret_cast<const v4i *>(stage + row * 32 + (threadIdx.x & 3) * 8);
          uint16_t *dst = p.out + int64_t(row) * p.ldo + n0;
          if (n0 + 8 <= p.N) {
            *reinterpret_cast<v4i *>(dst) = d;
          } else {
            const int w[4] = {d.x, d.y, d.z, d.w};
#pragma unroll
            for (int e = 0; e < 8; ++e)
              if (n0 + e < p.N) dst[e] = static_cast<uint16_t>(static_cast<uint32_t>(w[e >> 1]) >> (16 * (e & 1)));
          }
        }
      }
    }
  };

  // ---- the stream
  constexpr int NB = 3;  // (4 and 6 register sets: slower, they cost occupancy)
  Buf buf[NB];
  int slab = blockIdx.x, c = wave;  // the item being multiplied
  slab_begin(slab);
  static_for<NB - 1>([&](auto I) __attribute__((always_inline)) { issue(buf[I.value]); });
  if constexpr (XLDS) {
    // The copy of the token rows (up to 128 KB out of L2) is requested BEHIND the first weight chunks: issuing it
    // takes the workgroup about a microsecond, in which the weight requests are already on their way to HBM.
    __builtin_amdgcn_sched_barrier(0);
    copy_token_rows();
    // every wave's share of the token rows has landed (with the first weight chunks)
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    __syncthreads();
  }
  while (slab < slabs) {  // uniform over the workgroup: all waves see the same slab sequence
    static_for<NB>([&](auto I) __attribute__((always_inline)) {
      if (slab >= slabs) return;
      constexpr int i = I.value;
      issue(buf[(i + NB - 1) % NB]);
      multiply(buf[i], c);
      c += WAVES;
      if (c >= nchunks) {
        slab_end(slab);
        c = wave;
        slab += stride;
        slab_begin(slab);
      }
    });
  }
}

}  // namespace quik
