// Internals shared by the translation units of libkm_kernels: the error slot behind
// km_last_error() and the post-launch check.
#pragma once
#include <hip/hip_runtime.h>

#include "../../include/km_kernels.h"

int km_fail(int code, const char* message);
int km_check_launch(const char* where);

namespace km {
int gemm_num_configs();
int gemm_config_desc(int config, char* buf, int len);
int wo_num_configs();
int wo_config_desc(int config, char* buf, int len);
int blocks_gemm_num_configs();
int blocks_gemm_config_desc(int config, char* buf, int len);
// the 256 x 256 fp8 GEMM on the 32x32x64 MFMA (km_gemm_fp8_w32.hip)
int gemm_w32(bool mx, bool packed, int out_dtype, const void* a, const void* as, const void* b, const void* bs,
             const float* sa, const float* sb, const void* bias, void* c, int M, int N, int K, int scale_vectors,
             hipStream_t st);
}  // namespace km
