// Weight-only input-gradient kernels for f16 activations, int8 codes (see km_wo_dgrad.inc).
#define KM_WO_DT KM_F16
#define KM_WO_PART kWoPartI8
#include "km_wo_dgrad.inc"
