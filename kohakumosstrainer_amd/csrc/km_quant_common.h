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

// 8 values (one 128-bit load) -> 8 fp32
template <int DT>
__device__ __forceinline__ void widen8(const uint4& raw, float (&f)[8]) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = widen<DT>(w[i] & 0xFFFFu);
    f[2 * i + 1] = widen<DT>(w[i] >> 16);
  }
}

// ---- fp32-scale recipes (per row, per tensor) ---------------------------------------------------
// s = max(amax, 1e-12) / 448 and q = e4m3(clamp(x / s)), both IEEE fp32 divisions (reference
// formats.py:41-45).
__device__ __forceinline__ uint32_t wave_max(uint32_t m) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const uint32_t o = (uint32_t)__shfl_xor((int)m, off);
    m = o > m ? o : m;
  }
  return m;
}

// Codes of a row (tensor) whose amax is infinite or NaN, where clamp-and-convert instructions and the
// reference's host arithmetic part ways. Scale inf: finite x / inf is a signed zero, inf / inf
// is NaN. Scale NaN: every quotient is NaN; the reference's host division hands back the
// scale's NaN (code 0x7F) unless x is a NaN itself (code 0xFF, as for inf / inf).
template <int DT>
__device__ __forceinline__ uint32_t nonfinite_code(uint32_t h, bool nan_row) {
  const uint32_t a = h & 0x7FFFu;
  if (nan_row) return a > inf16<DT>() ? 0xFFu : 0x7Fu;
  return a == inf16<DT>() ? 0xFFu : (h >> 8) & 0x80u;
}

// x / s as the IEEE division rounds it, from r = RN(1 / s): a product and two fused
// corrections (each takes the exact remainder x - s q and adds remainder * r), the sign of x put
// back for zeros. With r correctly rounded the second correction rounds correctly whenever the
// first leaves q within one unit of the quotient; results differ from the division only far
// below 2^-11, where every code is a signed zero. The GPU tests compare the kernels built on it
// with the dividing element-wise kernels on every (amax, x) pair of 16-bit patterns.
__device__ __forceinline__ float quotient(float x, float s, float r) {
  float q = x * r;
  q = __builtin_fmaf(__builtin_fmaf(-s, q, x), r, q);
  q = __builtin_fmaf(__builtin_fmaf(-s, q, x), r, q);
  return __builtin_copysignf(q, x);
}

// codes of the eight values of one 128-bit load; r = RN(1 / s)
template <int DT>
__device__ __forceinline__ uint2 divided_codes8(const uint4& raw, float s, float r, bool finite, bool nan_row) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
  uint32_t out[2];
  if (finite) {
    float f[8];
    widen8<DT>(raw, f);
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = __builtin_amdgcn_fmed3f(quotient(f[i], s, r), -448.0f, 448.0f);
    out[0] = cvt4_f32(f[0], f[1], f[2], f[3], 1.0f);
    out[1] = cvt4_f32(f[4], f[5], f[6], f[7], 1.0f);
  } else {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      out[i] = nonfinite_code<DT>(w[2 * i] & 0xFFFFu, nan_row) | (nonfinite_code<DT>(w[2 * i] >> 16, nan_row) << 8) |
               (nonfinite_code<DT>(w[2 * i + 1] & 0xFFFFu, nan_row) << 16) | (nonfinite_code<DT>(w[2 * i + 1] >> 16, nan_row) << 24);
    }
  }
  return make_uint2(out[0], out[1]);
}

template <int DT>
__device__ __forceinline__ uint32_t divided_code1(uint32_t h, float s, bool finite, bool nan_row) {
  if (!finite) return nonfinite_code<DT>(h, nan_row);
  const float d = __builtin_amdgcn_fmed3f(__fdiv_rn(widen<DT>(h), s), -448.0f, 448.0f);
  return cvt4_f32(d, 0.f, 0.f, 0.f, 1.0f) & 0xFFu;
}

// scale from the largest 16-bit absolute-value pattern of a row
template <int DT>
__device__ __forceinline__ float scale_of_amax16(uint32_t m16) {
  if (m16 > inf16<DT>()) return bits_f32(0x7FC00000u);
  const uint32_t ab = widen_bits<DT>(m16);
  return __fdiv_rn(bits_f32(ab > kAmaxFloorBits ? ab : kAmaxFloorBits), 448.0f);
}

// the same from the fp32 bits of an amax
__device__ __forceinline__ float scale_of_amax_bits(uint32_t ab) {
  if (ab > kInfBits) return bits_f32(0x7FC00000u);
  return __fdiv_rn(bits_f32(ab > kAmaxFloorBits ? ab : kAmaxFloorBits), 448.0f);
}

}  // namespace km
