// Column map: the outlier split of one layer in the compact form the quantize kernels (and the weight
// repacking of the 6-bit path) read.  Built on the device by quik_colmap_build.
#pragma once
#include <stdint.h>

#include "common.h"

namespace quik {

// column map layout: [src_col: num_int idx][fp_col: num_fp idx][mask: ceil(cols/32) u32]
//                    [grp: ceil(cols/8) u32][dirty: min(num_fp, ceil(cols/8)) u32][dirty_grp: same count, u16]
//                    [kperm: num_int u16][patch: num_fp u32]
//                    [unit: ceil(num_int/16) u16][gather_unit: num_fp u16][gather_cols: num_fp x 16 u16][flags: 4 u32]
// idx is uint16_t when cols <= 65536, else uint32_t.  Section offsets are 16-byte aligned.
// A "group" is 8 consecutive source columns (one 16-byte load).  A group without outliers is
// clean, one with outliers is dirty; dirty groups are numbered in ascending order (slots).
//   grp[g]   clean: (destination column of the group's first element) << 8
//            dirty: (slot << 8) | mask byte (bit e set = column 8g+e is an outlier)
//   dirty[s] (destination column of the group's first non-outlier element) << 8 | mask byte
//   dirty_grp[s] the group index of dirty group s
//   flags[0] bit 0: int_indices ascending, the two lists partition the columns and the shape
//            fits the streaming kernel;  flags[1] = number of dirty groups.
//   flags[0] bit 1: the in-place order below exists; flags[2] = its number of holes.
//   flags[3] = number of gathered units (below), when the map streams and num_int % 16 == 0.
// grp, dirty, dirty_grp, kperm, patch, unit, gather_unit and gather_cols exist only when cols <= kStreamMaxCols.
//
// Units (int8 operand buffers in tile order): unit u is the 16 integer columns int_indices[16 u .. 16 u + 15], one
// 16-byte chunk of a row of the buffer.
//   unit[u]          the first of those columns when the 16 are consecutive source columns, else 0xFFFF
//   gather_unit[i]   the i-th unit (ascending) whose columns are not consecutive; at most one per outlier column
//   gather_cols[i]   its 16 source columns
//
// In-place order of the integer columns (operand buffers of the 6-bit path).  With num_int and num_fp
// multiples of 32, the first num_int source columns keep their places: position k holds source column k.
// Outlier columns among them leave holes; hole i (ascending) is filled by the i-th integer column of
// the tail [num_int, cols) (ascending), of which there are exactly as many.  A quantize kernel that works
// in this order never shifts data: it overwrites the holes of a row with their fillers and is done.
//   [kperm: num_int u16]  position k -> index of its column in ascending int_indices (the column of
//                         the packed weights that belongs at position k)
//   [patch: num_fp u32]   hole column | filler column << 16, flags[2] entries
struct ColmapLayout {
  bool idx16;
  int64_t off_fp, off_mask, off_grp, off_dirty, off_slot, off_kperm, off_patch, off_unit, off_gunit, off_gcols, off_flags,
      bytes;
};

__host__ __device__ inline int64_t align16(int64_t v) { return (v + 15) & ~int64_t(15); }

// Streaming (source-order) quantisation needs ascending int_indices, whole 16-byte chunks and at
// most kStreamMaxCols columns (16 chunks per thread held in registers).
constexpr int64_t kStreamMaxCols = 32768;

__host__ __device__ inline int64_t max_dirty_groups(int64_t cols, int64_t num_fp) {
  const int64_t groups = (cols + 7) / 8;
  return num_fp < groups ? num_fp : groups;
}

__host__ __device__ inline ColmapLayout colmap_layout(int64_t cols, int64_t num_int, int64_t num_fp) {
  ColmapLayout l;
  l.idx16 = cols <= 65536;
  const int64_t isz = l.idx16 ? 2 : 4;
  l.off_fp = align16(num_int * isz);
  l.off_mask = l.off_fp + align16(num_fp * isz);
  l.off_grp = l.off_mask + align16(((cols + 31) / 32) * 4);
  const bool stream = cols <= kStreamMaxCols;
  l.off_dirty = l.off_grp + align16(stream ? ((cols + 7) / 8) * 4 : 0);
  l.off_slot = l.off_dirty + align16(stream ? max_dirty_groups(cols, num_fp) * 4 : 0);
  l.off_kperm = l.off_slot + align16(stream ? max_dirty_groups(cols, num_fp) * 2 : 0);
  l.off_patch = l.off_kperm + align16(stream ? num_int * 2 : 0);
  l.off_unit = l.off_patch + align16(stream ? num_fp * 4 : 0);
  l.off_gunit = l.off_unit + align16(stream ? ((num_int + 15) / 16) * 2 : 0);
  l.off_gcols = l.off_gunit + align16(stream ? num_fp * 2 : 0);
  l.off_flags = l.off_gcols + (stream ? num_fp * 32 : 0);
  l.bytes = l.off_flags + 16;
  return l;
}

}  // namespace quik
