// Operand formats of the GEMMs that read their operands in tile order.
//
// 6-bit operand format of the int4 GEMM on the E2M3 matrix-core path (consumer: gemm_fp6.h).
//
// A level L = code + 8 (0 .. 15) is stored as a 6-bit field holding L: as an E2M3 number that is
// L / 8.  32 fields make a 24-byte fragment, element e in bits [6 e, 6 e + 6): a 16-byte head and
// an 8-byte tail.  One MFMA k-step covers 64 elements, fragment h = 0 / 1 of the step.
//
// The buffer is stored in the order the GEMM copies it into LDS, so that every wave-wide copy
// (64 lanes x 16 bytes) reads one contiguous, 1 KB aligned kilobyte: whole cache lines, each
// fetched exactly once per tile.  Rows are grouped in blocks of 64; unit (block B, step s) is 3 KB:
//   [0, 1024)     heads of rows 0..31 of the block: row r at 32 r, fragment h in 16-byte slot
//                 h ^ ((r >> 3) & 1)  (the slot swap keeps 16 consecutive rows of one fragment in 16
//                 different 16-byte bank groups of the 64-bank LDS)
//   [1024, 2048)  the same for rows 32..63
//   [2048, 3072)  tails: fragment h of row q (0..63) at 512 h + 8 q
// Element order along K: the in-place order of the column map (colmap.h): position k holds source column k of
// the activation, holes (outlier columns) filled by the integer columns of the tail; the weights are packed in
// the same order (the column map's kperm table), so the order cancels in the products.
// The outlier columns (fp16 / bf16, 16 per step t, i.e. two 16-byte chunks c per row and step) follow as
// further units of the same size whose third kilobyte is unused:
//   [0, 1024) rows 0..31, [1024, 2048) rows 32..63, row r at 32 r, chunk c in slot c ^ ((r >> 3) & 1).
// A block's units are contiguous: K / 64 integer steps, then F / 16 outlier steps, so the GEMM walks one
// pointer per block through all its steps.  The buffer ends with one int32 per row: the sum of the row's
// levels.
// Rows of the last block beyond the matrix are never written; any bit pattern is a finite E2M3
// or half value times results that are never stored.
#pragma once
#include "common.h"

namespace quik {

struct Fp6Layout {
  int64_t blocks, steps, fsteps, block_bytes, sums_off, bytes;
};
__host__ __device__ inline Fp6Layout fp6_layout(int64_t rows, int64_t K, int64_t F) {
  Fp6Layout l;
  l.blocks = (rows + 63) / 64;
  l.steps = K / 64;
  l.fsteps = F / 16;
  l.block_bytes = (l.steps + l.fsteps) * 3072;
  l.sums_off = l.blocks * l.block_bytes;
  l.bytes = l.sums_off + rows * 4;
  return l;
}

__host__ __device__ inline int64_t fp6_head_offset(const Fp6Layout &l, int64_t row, int64_t step, int h) {
  return (row >> 6) * l.block_bytes + step * 3072 + ((row >> 5) & 1) * 1024 + (row & 31) * 32 +
         ((h ^ ((row >> 3) & 1)) << 4);
}
__host__ __device__ inline int64_t fp6_tail_offset(const Fp6Layout &l, int64_t row, int64_t step, int h) {
  return (row >> 6) * l.block_bytes + step * 3072 + 2048 + h * 512 + (row & 63) * 8;
}
// 16-byte chunk c (8 values) of outlier step t
__host__ __device__ inline int64_t fp6_outlier_offset(const Fp6Layout &l, int64_t row, int64_t t, int c) {
  return fp6_head_offset(l, row, l.steps + t, c);
}

// ---- int8 operands in the same order (consumer: gemm_tile8.h): unit (block B, step s) is 2 KB, a step is 32
// int8 elements (or 16 fp16 / bf16 outlier values) = 32 bytes per row, two 16-byte chunks h per row
struct Tile8Layout {
  int64_t blocks, steps, fsteps, block_bytes, bytes;
};
__host__ __device__ inline Tile8Layout tile8_layout(int64_t rows, int64_t K, int64_t F) {
  Tile8Layout l;
  l.blocks = (rows + 63) / 64;
  l.steps = K / 32;
  l.fsteps = F / 16;
  l.block_bytes = (l.steps + l.fsteps) * 2048;
  l.bytes = l.blocks * l.block_bytes;
  return l;
}
// 16-byte chunk h of step `step` (integer steps first, then outlier steps) of row `row`
__host__ __device__ inline int64_t tile8_offset(const Tile8Layout &l, int64_t row, int64_t step, int h) {
  return (row >> 6) * l.block_bytes + step * 2048 + ((row >> 5) & 1) * 1024 + (row & 31) * 32 +
         ((h ^ ((row >> 3) & 1)) << 4);
}

// 4 levels (at most 63 each) in the bytes of w -> 24 bits, 6 per level: two byte dot products with the
// weights (1, 64) give b0 + 64 b1 and b2 + 64 b3, one shift-or joins them
__device__ __forceinline__ uint32_t fp6_squeeze4(uint32_t w) {
  const uint32_t lo = __builtin_amdgcn_udot4(w, 0x00004001u, 0u, false);
  const uint32_t hi = __builtin_amdgcn_udot4(w, 0x40010000u, 0u, false);
  return lo | (hi << 12);
}

// 32 levels, one per byte of b[0..7] in element order, -> the fragment's 6 dwords (head: 0..3, tail: 4..5)
__device__ __forceinline__ void fp6_pack_fragment(const uint32_t (&b)[8], uint32_t (&out)[6]) {
  uint32_t t[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) t[i] = fp6_squeeze4(b[i]);  // 24 bits each
  out[0] = t[0] | (t[1] << 24);
  out[1] = (t[1] >> 8) | (t[2] << 16);
  out[2] = (t[2] >> 16) | (t[3] << 8);
  out[3] = t[4] | (t[5] << 24);
  out[4] = (t[5] >> 8) | (t[6] << 16);
  out[5] = (t[6] >> 16) | (t[7] << 8);
}

// writes fragment f = 2 step + h of row `row` into an operand buffer
__device__ __forceinline__ void fp6_store_fragment(uint8_t *buf, const Fp6Layout &l, int64_t row, int64_t f,
                                                   const uint32_t (&o)[6]) {
  *reinterpret_cast<uint4 *>(buf + fp6_head_offset(l, row, f >> 1, f & 1)) = make_uint4(o[0], o[1], o[2], o[3]);
  *reinterpret_cast<uint2 *>(buf + fp6_tail_offset(l, row, f >> 1, f & 1)) = make_uint2(o[4], o[5]);
}

}  // namespace quik
