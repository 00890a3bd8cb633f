// Shared device/host helpers for libquik_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "quik_hip.h"

namespace quik {

// Last HIP error text, for quik_last_hip_error().
void set_last_hip_error(hipError_t e);
int check_launch();  // QUIK_OK or QUIK_ERR_LAUNCH after a kernel launch

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

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

// Round an fp32 value to the storage type and return it as fp32 again.
template <bool BF16>
__device__ __forceinline__ float round_storage(float f) {
  return to_f32<BF16>(from_f32<BF16>(f));
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float wave_min(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o, 64));
  return v;
}

}  // namespace quik
