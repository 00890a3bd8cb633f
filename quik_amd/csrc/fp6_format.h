// 6-bit operand format of the int4 GEMM on the E2M3 matrix-core path (consumer: gemm_fp6.h).
//
// A level L = code + 8 (0 .. 15) is stored as a 6-bit field holding L: as an E2M3 number that is
// L / 8.  32 fields make a 24-byte fragment, element e in bits [6 e, 6 e + 6).  Fragment g (0..3)
// of 128-element block kb of row r keeps its first 16 bytes in heads[r][kb][16 g .. 16 g + 16)
// and its last 8 bytes in tails[kb][g][r] (plane-major, rows padded to a multiple of 256 so that
// a tile's 128-row loads never leave the plane); the buffer ends with one int32 per row, the sum
// of the row's levels.
#pragma once
#include "common.h"

namespace quik {

struct Fp6Layout {
  int64_t rows_pad, kblocks, tails_off, sums_off, bytes;
};
__host__ __device__ inline Fp6Layout fp6_layout(int64_t rows, int64_t K) {
  Fp6Layout l;
  l.rows_pad = (rows + 255) / 256 * 256;
  l.kblocks = K / 128;
  l.tails_off = (rows * l.kblocks * 64 + 255) / 256 * 256;
  l.sums_off = l.tails_off + l.kblocks * 4 * l.rows_pad * 8;
  l.bytes = l.sums_off + rows * 4;
  return l;
}

// 4 levels in the bytes of w -> 24 bits, 6 per level
__device__ __forceinline__ uint32_t fp6_squeeze4(uint32_t w) {
  return (w & 0x3Fu) | ((w >> 2) & 0xFC0u) | ((w >> 4) & 0x3F000u) | ((w >> 6) & 0xFC0000u);
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

// writes one fragment (index f = 4 kb + g of row `row`) into an operand buffer
__device__ __forceinline__ void fp6_store_fragment(uint8_t *buf, const Fp6Layout &l, int64_t row, int64_t f,
                                                   const uint32_t (&o)[6]) {
  *reinterpret_cast<uint4 *>(buf + row * l.kblocks * 64 + f * 16) = make_uint4(o[0], o[1], o[2], o[3]);
  *reinterpret_cast<uint2 *>(buf + l.tails_off + (f * l.rows_pad + row) * 8) = make_uint2(o[4], o[5]);
}

}  // namespace quik
