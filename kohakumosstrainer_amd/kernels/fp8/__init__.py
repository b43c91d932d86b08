"""fp8 / MXFP8 compute formats and the fp8 linear ops."""

from kohakumosstrainer_amd.kernels.fp8.formats import (  # noqa: F401
    RECIPES,
    dequantize,
    pack_mx,
    quantize,
    swizzle_mx,
)
