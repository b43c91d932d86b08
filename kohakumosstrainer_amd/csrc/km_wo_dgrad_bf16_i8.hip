// Weight-only input-gradient kernels for bf16 activations, int8 codes (see km_wo_dgrad.inc).
#define KM_WO_DT KM_BF16
#define KM_WO_PART kWoPartI8
#include "km_wo_dgrad.inc"
