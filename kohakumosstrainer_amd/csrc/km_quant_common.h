// Device helpers shared by the quantizer kernels and the GEMM that quantizes its activations in
// the tile loop: widening of 16-bit inputs, the hardware e4m3 conversions and the 16-bit abs-max.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "km_internal.h"
#include "km_numeric.h"

namespace km {

template <int DT>
__device__ __forceinline__ float widen(uint32_t h);
template <>
__device__ __forceinline__ float widen<KM_BF16>(uint32_t h) { return bits_f32(h << 16); }
template <>
__device__ __forceinline__ float widen<KM_F16>(uint32_t h) {
  return __half2float(__ushort_as_half((unsigned short)h));
}

// ---- hardware e4m3 conversion ----------------------------------------------------------------
// V_CVT_SCALEF32_PK_FP8_{BF16,F16,F32} divide by the power of two in the exponent field of the
// scale operand, round once to nearest even and, with MODE.FP16_OVFL set, saturate at +-448: the
// reference's clamp((x * 2^-e)).to(e4m3) in one instruction per two elements, checked against
// the software encoder on every 16-bit input pattern and every scale byte a block can get.
// The one difference is NaN, which the instruction turns into 0xFF whatever the sign;
// nan_fix() restores 0x7F | sign.
typedef short v2s __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef unsigned short v2us __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void saturating_conversions() {
  asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 23, 1), 1");  // FP16_OVFL, per wavefront
}
// 16-bit absolute-value bits above which a pattern is a NaN
template <int DT>
constexpr uint32_t inf16() { return DT == KM_BF16 ? 0x7F80u : 0x7C00u; }
// fp32 bits of a non-negative 16-bit pattern (monotonic, NaN patterns stay above infinity)
template <int DT>
__device__ __forceinline__ uint32_t widen_bits(uint32_t h) {
  if constexpr (DT == KM_BF16) return h << 16;
  else return f32_bits(__half2float(__ushort_as_half((unsigned short)h)));
}
// four codes from two dwords of packed 16-bit values (a.lo, a.hi, b.lo, b.hi)
template <int DT>
__device__ __forceinline__ uint32_t cvt4(uint32_t a, uint32_t b, float scale) {
  v2s r = {0, 0};
  if constexpr (DT == KM_BF16) {
    r = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(r, __builtin_bit_cast(v2bf, a), scale, false);
    r = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(r, __builtin_bit_cast(v2bf, b), scale, true);
  } else {
    r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(r, __builtin_bit_cast(v2h, a), scale, false);
    r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(r, __builtin_bit_cast(v2h, b), scale, true);
  }
  return __builtin_bit_cast(uint32_t, r);
}
// four codes from four fp32 values
__device__ __forceinline__ uint32_t cvt4_f32(float a, float b, float c, float d, float scale) {
  v2s r = {0, 0};
  r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(r, a, b, scale, false);
  r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(r, c, d, scale, true);
  return __builtin_bit_cast(uint32_t, r);
}
// codes of the two 16-bit values in `h` (bytes `shift`, `shift`+8 of `codes`): NaN -> 0x7F | sign
template <int DT>
__device__ __forceinline__ uint32_t nan_fix(uint32_t codes, uint32_t h, int shift) {
  if ((h & 0x7FFFu) > inf16<DT>()) codes = (codes & ~(0xFFu << shift)) | ((0x7Fu | ((h >> 8) & 0x80u)) << shift);
  if (((h >> 16) & 0x7FFFu) > inf16<DT>()) codes = (codes & ~(0xFF00u << shift)) | ((0x7Fu | ((h >> 24) & 0x80u)) << (shift + 8));
  return codes;
}
// largest 16-bit absolute-value pattern of the eight values of one 128-bit load
__device__ __forceinline__ uint32_t amax16x8(const uint4& raw) {
  const v2us a = __builtin_bit_cast(v2us, raw.x & 0x7FFF7FFFu), b = __builtin_bit_cast(v2us, raw.y & 0x7FFF7FFFu);
  const v2us c = __builtin_bit_cast(v2us, raw.z & 0x7FFF7FFFu), d = __builtin_bit_cast(v2us, raw.w & 0x7FFF7FFFu);
  const v2us m = __builtin_elementwise_max(__builtin_elementwise_max(a, b), __builtin_elementwise_max(c, d));
  return m.x > m.y ? m.x : m.y;
}

}  // namespace km
