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
from kohakumosstrainer_amd.quant.stored import attach_stored, load_quantized, quantized_state, read_record, save_quantized
from kohakumosstrainer_amd.quant.weights import QuantWeight, dequantize, quantize

__all__ = [
    "ComputeCache",
    "ComputeWeight",
    "QuantLinear",
    "QuantWeight",
    "attach_compute",
    "attach_stored",
    "default_filter",
    "dequantize",
    "load_quantized",
    "quantize",
    "quantize_model",
    "quantize_torch_linears",
    "quantized_state",
    "read_record",
    "save_quantized",
]
