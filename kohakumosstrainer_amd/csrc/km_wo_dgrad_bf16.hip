// Weight-only input-gradient kernels for bf16 activations (see km_wo_dgrad.inc).
#define KM_WO_DT KM_BF16
#include "km_wo_dgrad.inc"
