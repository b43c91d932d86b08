// One block-scaled MFMA per wavefront on operands laid out by the host: D = A * B (E8M0 block scales) + C.
// Built and run by record_mfma_block_sum.py to record what the instruction returns.
#include <hip/hip_runtime.h>
#include <stdint.h>
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
__global__ void mfma_cases(const v8i* a, const v8i* b, const int* sa, const int* sb, const v4f* c, v4f* d) {
  const size_t i = (size_t)blockIdx.x * 64 + threadIdx.x;
  d[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[i], b[i], c[i], 0, 0, 0, sa[i], 0, sb[i]);
}
extern "C" int run_cases(const void* a, const void* b, const void* sa, const void* sb, const void* c, void* d, int ncase, void* stream) {
  hipLaunchKernelGGL(mfma_cases, dim3(ncase), dim3(64), 0, (hipStream_t)stream, (const v8i*)a, (const v8i*)b, (const int*)sa, (const int*)sb, (const v4f*)c, (v4f*)d);
  return (int)hipGetLastError();
}
