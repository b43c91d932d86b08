// Weight-only input-gradient kernels for bf16 activations, e4m3 codes, E8M0 or 128 x 128 block scales (see km_wo_dgrad.inc).
#define KM_WO_DT KM_BF16
#define KM_WO_PART kWoPartE4m3Blocks
#include "km_wo_dgrad.inc"
