"""Quantized frozen base weights (int8 / fp8 weight-only) and fp8 / MXFP8 compute (frozen
bases and trainable caches) for MossLinear and plain nn.Linear."""

from kohakumosstrainer_amd.quant.compute import ComputeCache, ComputeWeight
from kohakumosstrainer_amd.quant.convert import (
    QuantLinear,
    attach_compute,
    default_filter,
    quantize_model,
    quantize_torch_linears,
)
from kohakumosstrainer_amd.quant.weights import QuantWeight, dequantize, quantize

__all__ = [
    "ComputeCache",
    "ComputeWeight",
    "QuantLinear",
    "QuantWeight",
    "attach_compute",
    "default_filter",
    "dequantize",
    "quantize",
    "quantize_model",
    "quantize_torch_linears",
]
