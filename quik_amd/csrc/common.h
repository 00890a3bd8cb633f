// Shared device/host helpers for libquik_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "quik_hip.h"

namespace quik {

// Last HIP error text, for quik_last_hip_error().
void set_last_hip_error(hipError_t e);
int check_launch();  // QUIK_OK or QUIK_ERR_LAUNCH after a kernel launch
int num_cus();       // compute units of the GPU (asked once per process; 256 when no device answers)

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

// runtime.hip: flags word of a column map (colmap.h: bit 0 = streams, bit 1 = in-place order), copied from the
// device once per (address, shape) and remembered; colmap_forget drops what is known about an address.
// QUIK_ERR_COLMAP when the word is not known yet and `st` is being captured (no synchronisation possible there).
constexpr uint32_t kColmapStreams = 1u, kColmapInPlace = 2u;
int colmap_flags(const void *colmap, int64_t cols, int64_t num_int, int64_t num_fp, hipStream_t st, uint32_t *flags);
// all four flag words of the map (flags, number of dirty groups, number of holes, reserved), same look-up
int colmap_words(const void *colmap, int64_t cols, int64_t num_int, int64_t num_fp, hipStream_t st, uint32_t (&out)[4]);
void colmap_forget(const void *colmap);
// QUIK_OK when the column map has all bits of `need` set, QUIK_ERR_COLMAP when not (or an error of colmap_flags)
inline int colmap_require(const void *colmap, int64_t cols, int64_t num_int, int64_t num_fp, hipStream_t st,
                          uint32_t need) {
  uint32_t flags = 0;
  if (int rc = colmap_flags(colmap, cols, num_int, num_fp, st, &flags)) return rc;
  return (flags & need) == need ? QUIK_OK : QUIK_ERR_COLMAP;
}

// gemm.hip: MixedQLinear forward for one or two token rows in ONE launch, the quantize inside the kernel
// (w_red == NULL: symmetric activations with scale = max |x| / sym_divisor, fp16 only).  Returns kChainNotHandled
// (below) for shapes it leaves to the two-launch path.
int gemv_forward_one_launch(const void *x, int dtype, int64_t rows, int64_t cols, const void *colmap, int64_t num_int,
                            int64_t num_fp, int bits, const void *qw, const void *s_col, const void *w_red,
                            const void *fp_w, const void *bias, int64_t N, void *out, float sym_divisor,
                            hipStream_t st);

// gemm.hip: integer GEMM + the fp16-arithmetic epilogue of the reference's fused ops in one launch (zero_row ==
// NULL: symmetric form).  Returns kChainNotHandled for shapes it leaves to the two-launch path.
constexpr int kChainNotHandled = 1;
int int_gemm_chain(const void *A, const void *B, const void *s_row, const void *s_col, const void *zero_row,
                   const void *w_red, uint16_t shift_bits, const void *y, int64_t M, int64_t N, int64_t K, int bits,
                   void *out, hipStream_t st);

// ---- storage types as 16-bit patterns --------------------------------------------------
// Half values are handled with the native _Float16 type; bfloat16 with explicit bit math
// so that every rounding is a visible round-to-nearest-even.

template <bool BF16>
__device__ __forceinline__ float to_f32(uint16_t v) {
  if constexpr (BF16) {
    return __uint_as_float(static_cast<uint32_t>(v) << 16);
  } else {
    return static_cast<float>(__builtin_bit_cast(_Float16, v));
  }
}

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if (f != f) return 0x7FC0u;
  u += 0x7FFFu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}

template <bool BF16>
__device__ __forceinline__ uint16_t from_f32(float f) {
  if constexpr (BF16) {
    return f32_to_bf16_bits(f);
  } else {
    return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
  }
}

// Two fp32 values -> two storage values in one dword (first value in the low half).  fp16: the packed
// convert instruction of gfx950, same round-to-nearest-even as the scalar one.
template <bool BF16>
__device__ __forceinline__ uint32_t pack2_from_f32(float a, float b) {
  if constexpr (BF16) {
    return static_cast<uint32_t>(f32_to_bf16_bits(a)) | (static_cast<uint32_t>(f32_to_bf16_bits(b)) << 16);
  } else {
    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
    typedef float float2_t __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(float2_t{a, b}, half2_t));
  }
}

// Round an fp32 value to the storage type and return it as fp32 again.
template <bool BF16>
__device__ __forceinline__ float round_storage(float f) {
  return to_f32<BF16>(from_f32<BF16>(f));
}

// Lane exchange inside a row of 16 lanes through the DPP path of the vector ALU (no LDS traffic).
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
constexpr int kDppSwap1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppSwap2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // lane i <-> 7 - i inside each group of 8
constexpr int kDppMirror = 0x140;      // lane i <-> 15 - i inside each row of 16

// Wave-wide reductions; every lane of the wave must be active.  Four DPP steps make each row of 16
// uniform, the four rows are then combined through scalar registers.
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_move<kDppSwap1>(v));
  v = fmaxf(v, dpp_move<kDppSwap2>(v));
  v = fmaxf(v, dpp_move<kDppHalfMirror>(v));
  v = fmaxf(v, dpp_move<kDppMirror>(v));
  const int b = __builtin_bit_cast(int, v);
  const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0));
  const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
  const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32));
  const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
  return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}
__device__ __forceinline__ float wave_min(float v) {
  v = fminf(v, dpp_move<kDppSwap1>(v));
  v = fminf(v, dpp_move<kDppSwap2>(v));
  v = fminf(v, dpp_move<kDppHalfMirror>(v));
  v = fminf(v, dpp_move<kDppMirror>(v));
  const int b = __builtin_bit_cast(int, v);
  const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0));
  const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
  const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32));
  const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
  return fminf(fminf(r0, r1), fminf(r2, r3));
}

// integer sum over the wave (every lane active), same scheme
template <int CTRL>
__device__ __forceinline__ int dpp_move_i(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, false);
}
__device__ __forceinline__ int wave_sum(int v) {
  v += dpp_move_i<kDppSwap1>(v);
  v += dpp_move_i<kDppSwap2>(v);
  v += dpp_move_i<kDppHalfMirror>(v);
  v += dpp_move_i<kDppMirror>(v);
  return __builtin_amdgcn_readlane(v, 0) + __builtin_amdgcn_readlane(v, 16) + __builtin_amdgcn_readlane(v, 32) +
         __builtin_amdgcn_readlane(v, 48);
}

// ---- direct global -> LDS copies ---------------------------------------------------------
// One wave-wide 64 x 16-byte copy global -> LDS: lane i reads 16 bytes at sbase + voff_i and
// they land at LDS address m0 + 16 i.  sbase (scalar) and m0 are wave-uniform, so advancing K
// costs scalar adds only and a load is two instructions (s_mov m0, global_load_lds).  Written
// as inline assembly so that the outstanding-load count stays under this file's control: the
// loop waits with vmcnt(loads per stage), leaving the newest stage in flight across the barrier.
// (s_nop 0: one wait state between the scalar write of m0 and the copy that reads it, which the compiler
// keeps for its own LDS copies on this generation and cannot see inside an asm statement.  m0 is declared
// clobbered; the "memory" clobber orders the statement against the compiler's own LDS and global accesses.)
__device__ __forceinline__ void dma_load16(const uint8_t *sbase, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(voff), "s"(sbase) : "memory", "m0");
}

__device__ __forceinline__ uint32_t lds_address(const void *p) {
  return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) void *)p));
}

// s_waitcnt immediate for "vmcnt <= n", every other counter unconstrained (gfx9 encoding)
constexpr int vmcnt_imm(int n) { return (n & 0xF) | ((n >> 4) << 14) | 0x0F70; }

}  // namespace quik
