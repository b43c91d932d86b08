"""Quantized frozen base weights (int8 / fp8 weight-only) and fp8 / MXFP8 compute weights for
MossLinear and plain nn.Linear. Names resolve on first use, so importing the package does not
yet register any operator."""

import importlib

_HOME = {
    "compute": ("ComputeCache", "ComputeWeight"),
    "convert": ("QuantLinear", "attach_compute", "default_filter", "quantize_model", "quantize_torch_linears"),
    "stored": ("attach_stored", "load_quantized", "quantized_state", "read_record", "save_quantized"),
    "text": ("GroupQuantLinear", "linear_fate", "quantize_text_linears", "quantizes"),
    "weights": ("QuantWeight", "dequantize", "quantize"),
}
_WHERE = {name: module for module, names in _HOME.items() for name in names}
__all__ = sorted(_WHERE)


def __getattr__(name):
    if name in _WHERE:
        value = getattr(importlib.import_module(f"{__name__}.{_WHERE[name]}"), name)
        globals()[name] = value
        return value
    if name in _HOME:
        return importlib.import_module(f"{__name__}.{name}")
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")


def __dir__():
    return sorted(set(globals()) | set(__all__))
