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
}  // namespace km
