// Group Hadamard rotation (ConvRot) for gfx950: y = x . blockdiag(H_g) over the last axis,
// H_g the normalised Kronecker power of H4 = [[1,1,1,-1],[1,1,-1,1],[1,-1,1,1],[-1,1,1,1]],
// g = 4^j in {4, 16, 64, 256, 1024}. A bandwidth kernel: 2 bytes read and 2 written per element.
//
// Arithmetic follows the reference's butterfly form (src/kohakumoss_kernels/hadamard.py:71-82,
// the Triton kernel backends/triton/hadamard.py:28-49): j fp32 stages of 4-point butterflies
// y_k = ((x0 + x1) + x2) + x3 - 2 x_(3-k), the stage of the most significant base-4 digit of the
// index first, then one multiplication by 2^-j and one rounding to the 16-bit type. Every
// operation is a single fp32 rounding in a fixed order, so the result does not depend on the
// tiling (2 x is exact, so a fused multiply-subtract rounds the same).
//
// A workgroup of 256 lanes owns 4096 consecutive elements (whole groups, rows are contiguous):
// it loads them with 128-bit loads, keeps them as fp32 in LDS and runs the stages two at a time,
// each lane holding a 4 x 4 block of the two digits in registers (an odd j starts with one stage
// alone); the last pass leaves a lane with 16 consecutive elements, stored with 128-bit stores.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "km_hadamard_common.h"
#include "km_internal.h"
#include "km_numeric.h"

namespace km {

constexpr int kHadTile = 4096;
constexpr int kHadThreads = 256;

// J = log4(group)
template <int DT, int J>
__global__ __launch_bounds__(kHadThreads) void group_hadamard_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ y,
                                                                     int64_t numel) {
  constexpr int G = 1 << (2 * J);
  constexpr float kScale = 1.0f / (float)(1 << J);
  __shared__ __attribute__((aligned(16))) float tile[kHadTile];
  const int t = threadIdx.x;
  const int64_t base = (int64_t)blockIdx.x * kHadTile;
  // load: lane t takes elements [8 (t + 256 i), +8), i = 0, 1
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int e = 8 * (t + kHadThreads * i);
    uint4 raw = make_uint4(0, 0, 0, 0);
    if (base + e < numel) raw = *reinterpret_cast<const uint4*>(x + base + e);
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
    float4 lo, hi;
    lo.x = had_widen<DT>(w[0] & 0xFFFFu); lo.y = had_widen<DT>(w[0] >> 16); lo.z = had_widen<DT>(w[1] & 0xFFFFu); lo.w = had_widen<DT>(w[1] >> 16);
    hi.x = had_widen<DT>(w[2] & 0xFFFFu); hi.y = had_widen<DT>(w[2] >> 16); hi.z = had_widen<DT>(w[3] & 0xFFFFu); hi.w = had_widen<DT>(w[3] >> 16);
    *reinterpret_cast<float4*>(&tile[e]) = lo;
    *reinterpret_cast<float4*>(&tile[e + 4]) = hi;
  }
  __syncthreads();
  // an odd stage count starts with the first stage alone (stride G / 4): quad q = t + 256 i
  if constexpr (J % 2 == 1) {
    constexpr int S1 = G / 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int q = t + kHadThreads * i;
      const int first = (q / S1) * 4 * S1 + q % S1;
      float v0 = tile[first], v1 = tile[first + S1], v2 = tile[first + 2 * S1], v3 = tile[first + 3 * S1];
      h4(v0, v1, v2, v3);
      if constexpr (J == 1) {
        // S1 == 1: the quad is four consecutive elements and this was the only stage
        if (base + first < numel)
          *reinterpret_cast<uint2*>(y + base + first) = make_uint2(had_pack<DT>(v0 * kScale, v1 * kScale), had_pack<DT>(v2 * kScale, v3 * kScale));
      } else {
        // a lane writes back the positions it read (no other lane touches them in this pass)
        tile[first] = v0; tile[first + S1] = v1; tile[first + 2 * S1] = v2; tile[first + 3 * S1] = v3;
      }
    }
    if constexpr (J == 1) return;
    __syncthreads();
  }
  // double passes over the remaining stages, two at a time (strides 4 S and S); the last one has
  // S == 1 and leaves a lane with 16 consecutive elements
  constexpr int kDouble = J / 2;
  constexpr int kRest = J % 2 == 1 ? G / 4 : G;
#pragma unroll
  for (int p = 0; p < kDouble; ++p) {
    const int S = kRest >> (4 * (p + 1));
    const bool last = p == kDouble - 1;
    const int lo = t % S, top = t / S;
    const int first = top * 16 * S + lo;
    float v[4][4];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) v[a][b] = tile[first + (4 * a + b) * S];
#pragma unroll
    for (int b = 0; b < 4; ++b) h4(v[0][b], v[1][b], v[2][b], v[3][b]);
#pragma unroll
    for (int a = 0; a < 4; ++a) h4(v[a][0], v[a][1], v[a][2], v[a][3]);
    if (last) {
      if (base + first < numel) {
        uint32_t o[8];
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          o[2 * a] = had_pack<DT>(v[a][0] * kScale, v[a][1] * kScale);
          o[2 * a + 1] = had_pack<DT>(v[a][2] * kScale, v[a][3] * kScale);
        }
        uint4* dst = reinterpret_cast<uint4*>(y + base + first);
        dst[0] = make_uint4(o[0], o[1], o[2], o[3]);
        dst[1] = make_uint4(o[4], o[5], o[6], o[7]);
      }
      return;
    }
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) tile[first + (4 * a + b) * S] = v[a][b];
    __syncthreads();
  }
}

template <int DT>
static void launch_hadamard(int stages, const uint16_t* x, uint16_t* y, int64_t numel, hipStream_t st) {
  const dim3 grid((unsigned)((numel + kHadTile - 1) / kHadTile));
  switch (stages) {
    case 1: hipLaunchKernelGGL((group_hadamard_kernel<DT, 1>), grid, dim3(kHadThreads), 0, st, x, y, numel); break;
    case 2: hipLaunchKernelGGL((group_hadamard_kernel<DT, 2>), grid, dim3(kHadThreads), 0, st, x, y, numel); break;
    case 3: hipLaunchKernelGGL((group_hadamard_kernel<DT, 3>), grid, dim3(kHadThreads), 0, st, x, y, numel); break;
    case 4: hipLaunchKernelGGL((group_hadamard_kernel<DT, 4>), grid, dim3(kHadThreads), 0, st, x, y, numel); break;
    default: hipLaunchKernelGGL((group_hadamard_kernel<DT, 5>), grid, dim3(kHadThreads), 0, st, x, y, numel); break;
  }
}

}  // namespace km

using namespace km;

extern "C" int km_group_hadamard(const void* x, int64_t rows, int64_t cols, int dtype, int group, void* y, void* stream) {
  if (dtype != KM_BF16 && dtype != KM_F16) return km_fail(KM_ERR_ARG, "km_group_hadamard: dtype must be bf16 or f16");
  int stages = 0;
  for (int g = group; g > 1 && g % 4 == 0; g /= 4) ++stages;
  if (group < 4 || (1 << (2 * stages)) != group || stages > 5)
    return km_fail(KM_ERR_ARG, "km_group_hadamard: group must be 4, 16, 64, 256 or 1024");
  if (rows < 0 || cols < 0 || cols % group) return km_fail(KM_ERR_ARG, "km_group_hadamard: cols must be a non-negative multiple of the group");
  const int64_t numel = rows * cols;
  if (numel == 0) return KM_OK;
  if (!x || !y) return km_fail(KM_ERR_ARG, "km_group_hadamard: null pointer");
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) return km_fail(KM_ERR_UNSUPPORTED, "km_group_hadamard: operands must be 16-byte aligned");
  if ((numel + kHadTile - 1) / kHadTile > 0x7FFFFFFFll) return km_fail(KM_ERR_ARG, "km_group_hadamard: tensor too large");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == KM_BF16) launch_hadamard<KM_BF16>(stages, (const uint16_t*)x, (uint16_t*)y, numel, st);
  else launch_hadamard<KM_F16>(stages, (const uint16_t*)x, (uint16_t*)y, numel, st);
  return km_check_launch("km_group_hadamard");
}
