"""Model-side pieces of the quantized-linear path."""
