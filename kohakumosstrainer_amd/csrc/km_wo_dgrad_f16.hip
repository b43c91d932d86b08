// Weight-only input-gradient kernels for f16 activations (see km_wo_dgrad.inc).
#define KM_WO_DT KM_F16
#include "km_wo_dgrad.inc"
