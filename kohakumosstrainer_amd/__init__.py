"""MI355X (gfx950) native quantized linear: MXFP8 / per-tensor fp8 compute and int8 / fp8
weight-only linears as hand-written HIP kernels behind a C ABI (`native`), the per-op dispatch
and shape tuning table around them (`kernels`), and the nn.Linear-replacement modules
(`quant`, `model.linear`)."""

__version__ = "0.1.0"
