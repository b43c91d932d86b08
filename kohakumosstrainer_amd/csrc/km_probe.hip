// Measurement kernels (no counterpart in the reference; they compute nothing a caller needs).
//
// mfma_ceiling_kernel runs the block-scaled fp8 MFMA (V_MFMA_SCALE_F32_16X16X128_F8F6F4) out of
// registers only: one work-group of four wavefronts per compute unit, one wavefront per SIMD, each
// holding what a wavefront of the 256 x 256 GEMM tile holds (eight fragments of each operand, 64
// accumulator tiles in the 256 AGPRs) and issuing the same 64 MFMAs per trip with no load, no LDS
// access and no barrier between them. Every MFMA is independent of the 63 before it, so the matrix
// pipe never waits: the rate this loop reaches is what the card's clock and power management
// allow the matrix pipes under sustained load with these operands, the ceiling of any GEMM here.
#include <stdio.h>

#include "km_gemm_common.h"

namespace km {

__device__ __forceinline__ void probe_mfma(v4f& c, const v8i& a, const v8i& b, int sa, int sb) {
  asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:[0,0,0] op_sel_hi:[0,0,0]"
               : "+a"(c)
               : "v"(a), "v"(b), "v"(sa), "v"(sb));
}

// a_frags / b_frags: 64 lanes x 8 fragments x 32 bytes each (16 KiB), e4m3 codes; a wavefront's lane l
// takes bytes [(f * 64 + l) * 32, +32) of each as fragment f. sink: one fp32 per thread, written
// from the accumulators so that nothing is optimised away.
__global__ __launch_bounds__(256, 1) void mfma_ceiling_kernel(const v8i* __restrict__ a_frags, const v8i* __restrict__ b_frags,
                                                              float* __restrict__ sink, int trips) {
  const int lane = threadIdx.x & 63;
  v8i wf[8], xf[8];
#pragma unroll
  for (int f = 0; f < 8; ++f) {
    wf[f] = b_frags[f * 64 + lane];
    xf[f] = a_frags[f * 64 + lane];
  }
  v4f acc[8][8];
#pragma unroll
  for (int t = 0; t < 8; ++t)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      acc[t][j] = v4f{0.f, 0.f, 0.f, 0.f};
      asm volatile("" : "+a"(acc[t][j]));
    }
  const int unit = 0x7F7F7F7F;  // E8M0 bytes of 2^0
  for (int trip = 0; trip < trips; ++trip) {
#pragma unroll
    for (int t = 0; t < 8; ++t)
#pragma unroll
      for (int j = 0; j < 8; ++j) probe_mfma(acc[t][j], wf[t], xf[j], unit, unit);
  }
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
  float total = 0.f;
#pragma unroll
  for (int t = 0; t < 8; ++t)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float r;
      asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(r) : "a"(acc[t][j][0]));
      total += r;
    }
  sink[(size_t)blockIdx.x * 256 + threadIdx.x] = total;
}

}  // namespace km

using namespace km;

extern "C" int km_probe_mfma_ceiling(const void* a_frags, const void* b_frags, void* sink, int64_t sink_floats, int trips,
                                     int64_t* flop_out, void* stream) {
  if (!a_frags || !b_frags || !sink || !flop_out) return km_fail(KM_ERR_ARG, "km_probe_mfma_ceiling: null pointer");
  if (trips <= 0 || trips > (1 << 24)) return km_fail(KM_ERR_ARG, "km_probe_mfma_ceiling: trips out of range");
  if ((reinterpret_cast<uintptr_t>(a_frags) | reinterpret_cast<uintptr_t>(b_frags)) & 31)
    return km_fail(KM_ERR_UNSUPPORTED, "km_probe_mfma_ceiling: fragments must be 32-byte aligned");
  int device = 0, cus = 0;
  if (hipGetDevice(&device) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0)
    return km_fail(KM_ERR_LAUNCH, "km_probe_mfma_ceiling: device query failed");
  if (sink_floats < (int64_t)cus * 256) return km_fail(KM_ERR_ARG, "km_probe_mfma_ceiling: sink holds fewer than 256 floats per compute unit");
  hipLaunchKernelGGL(mfma_ceiling_kernel, dim3(cus), dim3(256), 0, (hipStream_t)stream, (const v8i*)a_frags, (const v8i*)b_frags,
                     (float*)sink, trips);
  // work-groups x wavefronts x trips x 64 MFMAs x (2 * 16 * 16 * 128) flop
  *flop_out = (int64_t)cus * 4 * trips * 64 * 65536;
  return km_check_launch("km_probe_mfma_ceiling");
}
