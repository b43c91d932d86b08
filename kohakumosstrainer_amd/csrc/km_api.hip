// Error reporting and the configuration catalogue of the C ABI.
#include <stdio.h>
#include <string.h>

#include "km_internal.h"

static thread_local char g_error[512] = "";

int km_fail(int code, const char* message) {
  snprintf(g_error, sizeof(g_error), "%s", message);
  return code;
}

int km_check_launch(const char* where) {
  hipError_t err = hipGetLastError();
  if (err == hipSuccess) return KM_OK;
  snprintf(g_error, sizeof(g_error), "%s: %s", where, hipGetErrorString(err));
  return KM_ERR_LAUNCH;
}

extern "C" int km_abi_version(void) { return 1; }
extern "C" const char* km_last_error(void) { return g_error; }

extern "C" int km_num_configs(int kernel) {
  switch (kernel) {
    case KM_KERNEL_GEMM_MX:
    case KM_KERNEL_GEMM_FP8: return km::gemm_num_configs();
    case KM_KERNEL_WO_FWD:
    case KM_KERNEL_WO_DGRAD: return km::wo_num_configs();
    case KM_KERNEL_GEMM_BLOCKS: return km::blocks_gemm_num_configs();
  }
  return km_fail(KM_ERR_ARG, "km_num_configs: unknown kernel");
}

extern "C" int km_config_desc(int kernel, int config, char* buf, int len) {
  if (!buf || len <= 0) return km_fail(KM_ERR_ARG, "km_config_desc: no buffer");
  switch (kernel) {
    case KM_KERNEL_GEMM_MX:
    case KM_KERNEL_GEMM_FP8: return km::gemm_config_desc(config, buf, len);
    case KM_KERNEL_WO_FWD:
    case KM_KERNEL_WO_DGRAD: return km::wo_config_desc(config, buf, len);
    case KM_KERNEL_GEMM_BLOCKS: return km::blocks_gemm_config_desc(config, buf, len);
  }
  return km_fail(KM_ERR_ARG, "km_config_desc: unknown kernel");
}
