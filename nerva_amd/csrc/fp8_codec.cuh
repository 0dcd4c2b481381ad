// FP8 e4m3fn (OCP: no infinities, 0x7f/0xff NaN, subnormal step 2^-9) codecs.
// Reference: f8_e4m3fn_bits_to_f32 (precision/bits.rs:87-104),
// f32_to_f8_e4m3fn_bits (crates/nerva-cuda/src/deepseek_quant/fp8.rs:18-72).
#pragma once

#include "nv_common.cuh"

namespace nv {

// Bit-level decode, valid on any target.
__device__ __forceinline__ float fp8_e4m3fn_to_f32_sw(uint32_t b) {
  const uint32_t sign = (b & 0x80u) << 24;
  const uint32_t em = b & 0x7fu;
  if (em == 0x7fu) return __uint_as_float(0x7fc00000u);
  if (em < 8u) return __uint_as_float(sign | __float_as_uint(static_cast<float>(em) * 0.001953125f));
  return __uint_as_float(sign | ((em << 20) + 0x3c000000u));
}

typedef float f32x2_t __attribute__((ext_vector_type(2)));

// Four packed e4m3fn bytes -> four floats with the gfx950 conversion
// instruction (v_cvt_pk_f32_fp8, OCP encoding on gfx950). An exhaustive GPU
// test compares all 256 codes against the bit-level decode above.
__device__ __forceinline__ void fp8x4_to_f32(uint32_t packed, float (&out)[4]) {
  const f32x2_t lo = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(packed), false);
  const f32x2_t hi = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(packed), true);
  out[0] = lo.x;
  out[1] = lo.y;
  out[2] = hi.x;
  out[3] = hi.y;
}

// RNE, saturate to +-448 (0x7e/0xfe), NaN -> 0x7f, signed zero preserved.
__device__ __forceinline__ uint8_t f32_to_fp8_e4m3fn(float value) {
  const uint32_t bits = __float_as_uint(value);
  const uint32_t sign = (bits >> 24) & 0x80u;
  const uint32_t abs_bits = bits & 0x7fffffffu;
  if (abs_bits > 0x7f800000u) return 0x7f;
  const float a = __uint_as_float(abs_bits);
  if (a > 448.0f) return static_cast<uint8_t>(sign | 0x7eu);
  if (a < 0.015625f) {
    const uint32_t quantum = static_cast<uint32_t>(rintf(a * 512.0f));  // ties-to-even
    return static_cast<uint8_t>(sign | quantum);
  }
  int exp32 = static_cast<int>(abs_bits >> 23) - 127;
  const uint32_t mant = abs_bits & 0x007fffffu;
  uint32_t q = mant >> 20;
  const uint32_t r = mant & 0x000fffffu;
  if (r > 0x80000u || (r == 0x80000u && (q & 1u) == 1u)) {
    q += 1;
    if (q == 8) {
      q = 0;
      exp32 += 1;
    }
  }
  return static_cast<uint8_t>(sign | ((static_cast<uint32_t>(exp32 + 7) << 3) | q));
}

}  // namespace nv
