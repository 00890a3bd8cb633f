// Per-row quantisation arithmetic shared by the quantize kernels (quantize.hip) and the single-launch decode forward
// (gemm_gemv.h): scale / zero / reciprocal of a row, the codes of a group of 8 columns, packed fp16 min / max.
#pragma once
#include "common.h"

namespace quik {

template <bool BF16>
struct RowQuant {
  float zero, scale, rcp;
  bool slow;
  uint16_t scale_bits, zero_bits;

  __device__ __forceinline__ void init(float mn, float mx, int bits) {
    if (!(mx >= mn)) {  // no non-NaN element in the row
      mn = mx = __builtin_nanf("");
    }
    const float range = mx - mn;
    const float s32 = fmaxf(range / static_cast<float>((1 << bits) - 1), 1e-6f);
    scale_bits = from_f32<BF16>(s32);
    zero_bits = from_f32<BF16>(mn);
    scale = to_f32<BF16>(scale_bits);
    zero = mn;
    rcp = 1.0f / scale;
    const float max_finite = BF16 ? 3.3895313892515355e38f : 65504.0f;
    slow = !(range <= max_finite) || !(scale >= 1e-20f);
  }

  // Symmetric activations (reference: experiments/qlinear.py:97-103): scale = fp16(max |x| / divisor), zero = 0.
  // `absmax_bits` is the largest |x| as an fp16 bit pattern (NaN patterns count as larger than infinity, so a NaN
  // in the row makes the scale NaN, as torch.max does).
  __device__ __forceinline__ void init_sym(uint32_t absmax_bits, float divisor) {
    const float absmax = to_f32<false>(static_cast<uint16_t>(absmax_bits));
    scale_bits = from_f32<false>(absmax / divisor);
    zero_bits = 0;
    scale = to_f32<false>(scale_bits);
    zero = 0.0f;
    rcp = 1.0f / scale;
    slow = !(scale >= 1e-6f) || !(absmax <= 65504.0f);
  }

  // same with the path chosen at compile time (callers branch once per row on `slow`)
  template <bool SLOW>
  __device__ __forceinline__ float quotient_t(uint16_t xbits) const {
    float d;
    if constexpr (BF16) {
      d = round_storage<true>(to_f32<true>(xbits) - zero);
    } else {
      const _Float16 dh = __builtin_bit_cast(_Float16, xbits) - static_cast<_Float16>(zero);
      d = static_cast<float>(dh);
    }
    float q;
    if constexpr (SLOW) {
      q = d / scale;
    } else {
      q = d * rcp;
      const float e = __builtin_fmaf(-q, scale, d);
      q = __builtin_fmaf(e, rcp, q);
    }
    return round_storage<BF16>(q);
  }

  // storage(storage(x - zero) / scale) as fp32
  __device__ __forceinline__ float quotient(uint16_t xbits) const {
    float d;
    if constexpr (BF16) {
      d = round_storage<true>(to_f32<true>(xbits) - zero);
    } else {
      const _Float16 dh = __builtin_bit_cast(_Float16, xbits) - static_cast<_Float16>(zero);
      d = static_cast<float>(dh);
    }
    float q;
    if (slow) {
      q = d / scale;
    } else {
      q = d * rcp;
      const float e = __builtin_fmaf(-q, scale, d);
      q = __builtin_fmaf(e, rcp, q);
    }
    return round_storage<BF16>(q);
  }

  // clamp(rne_int(t), 0, maxq), NaN -> 0, for maxq <= 255
  static __device__ __forceinline__ uint32_t to_level(float t, float maxq) {
    const float c = fminf(fmaxf(t, 0.0f), maxq);
    return __float_as_uint(c + 12582912.0f) & 0xFFu;  // 1.5 * 2^23: integer lands in the low mantissa bits
  }
};

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef float f2 __attribute__((ext_vector_type(2)));
typedef uint16_t u2 __attribute__((ext_vector_type(2)));

struct __attribute__((packed, aligned(1))) Bytes8 {
  uint32_t a, b;
};

// Codes of the two halves of word w in bytes 0 and 2 of the result (other bytes: don't care).
// The code is (level - 2^(BITS-1)) mod 256; for BITS == 4 only its low nibble is meaningful.
// SYM (fp16 only): symmetric codes, rne(fp16(x / scale)) kept modulo 256 without a clamp (reference:
// src/symmetric/symmetric.cu:6-61; NaN -> 0, +-infinity saturate as __half2int_rn does before the low bits are cut).
// (The v_fma_mix pairs below are plain VALU instructions; their output is early-clobber because the second
// instruction of a pair reads the inputs after the first has written its half: no wait-state hazard.)
template <int BITS, bool BF16, bool SLOW, bool SYM = false>
__device__ __forceinline__ uint32_t code_pair(uint32_t w, const RowQuant<BF16> &rq) {
  constexpr float kMaxQ = static_cast<float>((1 << BITS) - 1);
  constexpr uint32_t kBias = 1u << (BITS - 1);
  if constexpr (SYM) {
    static_assert(!BF16, "symmetric activations are fp16");
    const h2 d = __builtin_bit_cast(h2, w);
    h2 t;
    if constexpr (SLOW) {
      const f2 q = f2{static_cast<float>(d.x) / rq.scale, static_cast<float>(d.y) / rq.scale};
      t = __builtin_convertvector(q, h2);
    } else {
      uint32_t tb;
      asm("v_fma_mixlo_f16 %0, %1, %2, 0 op_sel_hi:[1,0,0]\n\t"
          "v_fma_mixhi_f16 %0, %1, %2, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]"
          : "=&v"(tb)
          : "v"(w), "v"(rq.rcp));
      t = __builtin_bit_cast(h2, tb);
    }
    // [-512, 511] holds every legitimate quotient (|q| <= divisor) unchanged, maps NaN to -512 and the infinities to
    // the ends; + 1536 lands in [1024, 2048), where one fp16 ulp is 1: the sum is rne(t) + 1536 and its low byte is
    // rne(t) mod 256 (0 for NaN and -infinity, 255 for +infinity: the low bits of the saturated integers)
    const _Float16 lo = static_cast<_Float16>(-512.0f), hi = static_cast<_Float16>(511.0f);
    t = __builtin_elementwise_min(__builtin_elementwise_max(t, h2{lo, lo}), h2{hi, hi});
    constexpr _Float16 magic = static_cast<_Float16>(1536);
    t = t + h2{magic, magic};
    return __builtin_bit_cast(uint32_t, t);
  } else if constexpr (BF16) {
    const uint32_t a = RowQuant<true>::to_level(rq.template quotient_t<SLOW>(static_cast<uint16_t>(w & 0xFFFFu)), kMaxQ);
    const uint32_t b = RowQuant<true>::to_level(rq.template quotient_t<SLOW>(static_cast<uint16_t>(w >> 16)), kMaxQ);
    return (a + kBias) | ((b + kBias) << 16);
  } else {
    const h2 x = __builtin_bit_cast(h2, w);
    const _Float16 zh = static_cast<_Float16>(rq.zero);
    const h2 d = x - h2{zh, zh};  // storage(x - zero), both halves
    h2 t;                         // storage(d / scale), or a value that rounds to the same level
    if constexpr (SLOW) {
      const f2 q = f2{static_cast<float>(d.x) / rq.scale, static_cast<float>(d.y) / rq.scale};
      t = __builtin_convertvector(q, h2);
    } else {
      // fp16(f32(d) * rcp) for both halves: the mixed-precision FMA reads an fp16 half and an fp32
      // register and writes an fp16 half, so the quotient costs one instruction per element
      uint32_t tb;
      asm("v_fma_mixlo_f16 %0, %1, %2, 0 op_sel_hi:[1,0,0]\n\t"
          "v_fma_mixhi_f16 %0, %1, %2, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]"
          : "=&v"(tb)
          : "v"(__builtin_bit_cast(uint32_t, d)), "v"(rq.rcp));
      t = __builtin_bit_cast(h2, tb);
    }
    // clamp to [0, maxq] (NaN -> 0), then + 1024 + 2^(BITS-1): in [1024, 2048) one fp16 ulp is 1, so the
    // sum is round-to-nearest-even(t) + 2^(BITS-1) and that integer sits in the low mantissa bits
    const _Float16 mq = static_cast<_Float16>(kMaxQ);
    t = __builtin_elementwise_min(__builtin_elementwise_max(t, h2{0, 0}), h2{mq, mq});
    constexpr _Float16 magic = static_cast<_Float16>(1024 + (1 << (BITS - 1)));
    t = t + h2{magic, magic};
    return __builtin_bit_cast(uint32_t, t);
  }
}

// 8 codes of one group as 8 bytes
template <int BITS, bool BF16, bool SLOW, bool SYM = false>
__device__ __forceinline__ uint2 group_codes(const uint4 &v, const RowQuant<BF16> &rq) {
  const uint32_t p0 = code_pair<BITS, BF16, SLOW, SYM>(v.x, rq), p1 = code_pair<BITS, BF16, SLOW, SYM>(v.y, rq);
  const uint32_t p2 = code_pair<BITS, BF16, SLOW, SYM>(v.z, rq), p3 = code_pair<BITS, BF16, SLOW, SYM>(v.w, rq);
  uint2 c;
  c.x = __builtin_amdgcn_perm(p1, p0, 0x06040200u);  // bytes 0, 2 of p0 then bytes 0, 2 of p1
  c.y = __builtin_amdgcn_perm(p3, p2, 0x06040200u);
  if constexpr (BITS == 4) {
    c.x &= 0x0F0F0F0Fu;
    c.y &= 0x0F0F0F0Fu;
  }
  return c;
}

// Packed fp16 min / max as single instructions.  (The compiler's own minnum / maxnum first quiet a possible
// signalling NaN with an extra v_pk_max x, x whenever it cannot prove that the operand is not one.)
// (Plain VALU instructions on the statement's own operands, not volatile: no wait-state hazard, and the compiler
// is free to schedule or drop them like any other arithmetic.)
__device__ __forceinline__ uint32_t pk_min_f16(uint32_t a, uint32_t b) {
  uint32_t r;
  asm("v_pk_min_f16 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
__device__ __forceinline__ uint32_t pk_max_f16(uint32_t a, uint32_t b) {
  uint32_t r;
  asm("v_pk_max_f16 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}

// The IEEE bit of the MODE register makes v_pk_min_f16 / v_pk_max_f16 answer a SIGNALLING NaN operand with a quiet
// NaN instead of the other operand, which would then be lost from a running minimum.  Kernels that use the two
// helpers above on raw input clear the bit for themselves: every NaN is skipped alike, as __hmin / __hmax and fminf
// skip it.  (Nothing else in these kernels depends on the bit: it only selects how signalling NaNs are treated.)
__device__ __forceinline__ void treat_all_nans_alike() {
  asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 9, 1), 0");
}

}  // namespace quik
