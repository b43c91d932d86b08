// Weight-only forward kernels for f16 activations (see km_wo_fwd.inc).
#define KM_WO_DT KM_F16
#include "km_wo_fwd.inc"
