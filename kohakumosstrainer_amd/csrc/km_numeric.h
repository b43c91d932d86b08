// Scalar numeric building blocks shared by every kernel: e4m3fn encoding, the MX block
// exponent and exact widenings. Pure integer / IEEE fp32 arithmetic with no HIP
// dependency, so the same functions compile for the device (hipcc) and for the host
// (g++), where the CPU tests check them bit by bit.
//
//   e4m3 rounding      reference src/kohakumoss_kernels/fp8/formats.py:44-45,98
//                      ("clamp to +-448, round once")
//   MX block exponent  reference src/kohakumoss_kernels/fp8/formats.py:55-61
//   2^-e from a byte   reference src/kohakumoss_kernels/fp8/formats.py:64-67
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define KM_HD __host__ __device__ __forceinline__
#else
#define KM_HD inline
#endif

namespace km {

constexpr uint32_t kAbsMask = 0x7FFFFFFFu;
constexpr uint32_t kInfBits = 0x7F800000u;
constexpr uint32_t kE4M3MaxBits = 0x43E00000u;   // 448.0f
constexpr uint32_t kMxAmaxFloorBits = 0x0DA24260u;  // 1e-30f
constexpr uint32_t kAmaxFloorBits = 0x2B8CBCCCu;    // 1e-12f

KM_HD uint32_t f32_bits(float f) { return __builtin_bit_cast(uint32_t, f); }
KM_HD float bits_f32(uint32_t u) { return __builtin_bit_cast(float, u); }

// Biased E8M0 byte (e + 127) of a block from the bits of its non-negative fp32 amax:
// amax = m * 2^E needs e = E - 8, one more when m > 1.75. Non-negative floats order
// like their bit patterns, so the 1e-30 floor is an integer max, and a NaN amax (bits
// above infinity) passes through it as it passes through a clamp.
KM_HD uint32_t mx_biased_exponent(uint32_t amax_bits) {
  uint32_t b = amax_bits > kMxAmaxFloorBits ? amax_bits : kMxAmaxFloorBits;
  uint32_t up = (b & 0x007FFFFFu) > 0x00600000u ? 1u : 0u;
  return (b >> 23) - 8u + up;  // >= 19 thanks to the floor
}

// Exact fp32 2^-(biased - 127) for biased in [0, 253].
KM_HD float mx_inverse_scale(uint32_t biased) { return bits_f32((254u - biased) << 23); }

// e4m3fn byte of an fp32 value: magnitude clamped to 448 (infinity included), rounded
// once to nearest with ties to the even code, subnormal codes below 2^-6, the input's
// sign bit kept (negative zero and negative underflow give 0x80), NaN -> 0x7F | sign.
KM_HD uint32_t e4m3_encode(float v) {
  uint32_t w = f32_bits(v);
  uint32_t sign = (w >> 24) & 0x80u;
  uint32_t a = w & kAbsMask;
  if (a > kInfBits) return sign | 0x7Fu;
  a = a < kE4M3MaxBits ? a : kE4M3MaxBits;
  uint32_t code;
  if (a >= (121u << 23)) {
    // normal e4m3: keep 3 of the 23 mantissa bits, round half to even; a carry moves
    // into the exponent field, which is what the next binade's first code needs
    uint32_t lsb = (a >> 20) & 1u;
    code = ((a + 0x7FFFFu + lsb) >> 20) - (120u << 3);
  } else {
    // below 2^-6 the codes count steps of 2^-9: adding 2^14 makes the fp32 adder round
    // to that step (ties to even), leaving the count in the low mantissa bits
    float r = bits_f32(a) + 16384.0f;
    code = f32_bits(r) - 0x46800000u;
  }
  return sign | code;
}

// Exact fp32 value of an e4m3fn byte (NaN bytes give NaN).
KM_HD float e4m3_decode(uint32_t code) {
  uint32_t sign = (code & 0x80u) << 24;
  uint32_t mag = code & 0x7Fu;
  if (mag == 0x7Fu) return bits_f32(sign | 0x7FC00000u);
  if (mag < 8u) return bits_f32(sign | f32_bits((float)mag * 0.001953125f));
  return bits_f32(sign | ((mag + (120u << 3)) << 20));
}

KM_HD float bf16_bits_to_f32(uint32_t h) { return bits_f32(h << 16); }

// fp32 -> bf16 bits, round to nearest even (NaN kept quiet).
KM_HD uint32_t f32_to_bf16_bits(float f) {
  uint32_t w = f32_bits(f);
  if ((w & kAbsMask) > kInfBits) return (w >> 16) | 0x40u;
  return (w + 0x7FFFu + ((w >> 16) & 1u)) >> 16;
}

}  // namespace km
