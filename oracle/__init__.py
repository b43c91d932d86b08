"""CPU oracle of the quantized-linear hot path. TEST INFRASTRUCTURE ONLY.

Everything under this directory restates, on the CPU with torch / numpy / plain C, what
the reference's eager (torch) path computes for the quantized linear: the fp8 / MXFP8
quantizers and dequantizers, the dequantize-then-matmul linear forward and input
gradient, the weight-only int8 / fp8 linear, the int8 compute linear, and the error statistics the reference's
tests judge a kernel by. Only `tests/`, `__graft_entry__.smoke()` and the
`cpu_baseline` leg of `bench.py` may import it, and only as the checker: the shipped
package never imports it and has no CPU fallback on a GPU.

How each function is pinned (independently of its own formula):

  formats.e4m3 rounding        full enumeration of the 256 e4m3fn codes, nearest value
                               with ties to the even code, saturation at 448
                               (tests/test_oracle_pins.py), all 65 536 bf16 patterns
  formats.mx_biased_exponent   definition "smallest e >= -127 with 2^e*448 >= amax"
                               by a loop in exact arithmetic; the reference tests'
                               known answers (amax 1.75 -> 119, 1.75(1+2^-7) -> 120,
                               all-zero block -> 19, and so 448*2^-130: the 1e-30 amax
                               floor makes byte 0 unreachable)
  formats.fp32_scale           correctly rounded fp32 division via numpy float32
  formats.quantize / dequantize  block-by-block application of the two above; q*scale
                               per element in fp64
  formats.swizzle_mx           the 32x4x4 index formula applied element by element
  linear.*                     fp64 matmul of the exactly dequantized operands
                               (tolerance, as the reference's own tests do)
  weights.quantize             np.rint half-to-even known answers, 2^-4 error bound
  int8.quantize_rows           the reference tests' half-to-even known answers and floor
                               scale; numpy float32 division and np.rint
  int8.int_mm                  Python-integer matrix product
  int8.forward / dgrad         an fp64 model of the scheme: exact agreement on inputs
                               that quantize without error, closeness elsewhere,
                               broken designs must fail (tests/test_oracle_int8.py)
  hadamard.*                   fp64 torch.kron construction, H H = I, exact equality on
                               integer inputs (tests/test_oracle_hadamard.py)
  mxq.c (C restatement)        bit-compared against formats.quantize on random,
                               edge-case and exhaustive bf16 inputs

No function here is "parity unpinned".
"""
