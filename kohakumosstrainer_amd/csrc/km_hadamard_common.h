// The 4-point butterfly of the group Hadamard rotation and the 16-bit conversions around it, shared
// by the rotation kernel and by the quantizer that rotates on the way in.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "km_internal.h"
#include "km_numeric.h"

namespace km {

__device__ __forceinline__ void h4(float& x0, float& x1, float& x2, float& x3) {
  const float total = ((x0 + x1) + x2) + x3;
  const float y0 = total - 2.0f * x3, y1 = total - 2.0f * x2, y2 = total - 2.0f * x1, y3 = total - 2.0f * x0;
  x0 = y0; x1 = y1; x2 = y2; x3 = y3;
}

template <int DT>
__device__ __forceinline__ float had_widen(uint32_t h) {
  if constexpr (DT == KM_BF16) return bits_f32(h << 16);
  else return __half2float(__ushort_as_half((unsigned short)h));
}
template <int DT>
__device__ __forceinline__ uint32_t had_narrow(float f) {
  if constexpr (DT == KM_BF16) return f32_to_bf16_bits(f);
  else return (uint32_t)__half_as_ushort(__float2half_rn(f));
}
template <int DT>
__device__ __forceinline__ uint32_t had_pack(float a, float b) { return had_narrow<DT>(a) | (had_narrow<DT>(b) << 16); }

}  // namespace km
