// Weight-only dequant-GEMMs (placeholder translation unit while the kernels are written).
#include "km_internal.h"

namespace km {
int wo_num_configs() { return 0; }
int wo_config_desc(int, char*, int) { return km_fail(KM_ERR_ARG, "config out of range"); }
}  // namespace km

extern "C" int km_wo_gemm_fwd(const void*, const void*, const float*, const void*, void*, int64_t, int64_t,
                              int64_t, int, int, int, void*) {
  return km_fail(KM_ERR_UNSUPPORTED, "km_wo_gemm_fwd: not built yet");
}
extern "C" int km_wo_gemm_dgrad(const void*, const void*, const float*, void*, int64_t, int64_t, int64_t, int,
                                int, int, void*) {
  return km_fail(KM_ERR_UNSUPPORTED, "km_wo_gemm_dgrad: not built yet");
}
