// Weight-only input-gradient kernels for f16 activations, e4m3 codes, one scale per row or tensor (see km_wo_dgrad.inc).
#define KM_WO_DT KM_F16
#define KM_WO_PART kWoPartE4m3Rows
#include "km_wo_dgrad.inc"
