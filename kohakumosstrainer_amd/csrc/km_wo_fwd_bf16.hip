// Weight-only forward kernels for bf16 activations (see km_wo_fwd.inc).
#define KM_WO_DT KM_BF16
#include "km_wo_fwd.inc"
