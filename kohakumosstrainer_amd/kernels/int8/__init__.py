"""int8 compute over frozen int8 weights: formats and the `int8_linear` op."""

from kohakumosstrainer_amd.kernels.int8.formats import INT8_MAX, col_major, int_mm, quantize_rows, row_scale  # noqa: F401
