/* Oracle (test infrastructure): plain C restatement of the reference's MXFP8 and
 * per-tensor e4m3 quantizers for bf16 input, written from the format definitions with
 * libm (frexpf / ldexpf / nearbyintf) rather than bit tricks, so that it is a second,
 * independent implementation next to oracle/formats.py.
 *
 *   reference src/kohakumoss_kernels/fp8/formats.py:55-61   block exponent
 *   reference src/kohakumoss_kernels/fp8/formats.py:94-99   mx codes
 *   reference src/kohakumoss_kernels/fp8/formats.py:44-52,77-79  per-tensor scale, codes
 *
 * Never linked into the shipped library; built by oracle/build.py into
 * oracle/_build/liboracle_mxq.so and loaded only by tests and bench.py's cpu_baseline.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static float bf16_to_f32(uint16_t h) {
  uint32_t w = (uint32_t)h << 16;
  float f;
  memcpy(&f, &w, 4);
  return f;
}

/* One rounding of a finite-or-not fp32 value to e4m3fn after clamping to +-448: ties go
 * to the even code, the sign survives a zero result, NaN keeps its sign and becomes 0x7F. */
uint8_t oracle_e4m3_from_f32(float v) {
  uint32_t w;
  memcpy(&w, &v, 4);
  uint8_t sign = (uint8_t)((w >> 24) & 0x80);
  if (v != v) return sign | 0x7F;
  float a = fabsf(v);
  if (a > 448.0f) a = 448.0f;
  if (a == 0.0f) return sign;
  int e;
  (void)frexpf(a, &e); /* a = m * 2^e, m in [0.5, 1) -> floor(log2 a) = e - 1 */
  int p = e - 1;
  if (p < -6) p = -6;                                /* subnormal codes share 2^-6's step */
  float steps = nearbyintf(ldexpf(a, 3 - p));        /* a / 2^(p-3), ties to even */
  if (steps >= 16.0f) { steps = 8.0f; p += 1; }      /* carried into the next binade */
  int n = (int)steps;
  if (n < 8) return sign | (uint8_t)n;               /* subnormal (p == -6) or zero */
  return sign | (uint8_t)(((p + 7) << 3) | (n - 8));
}

/* Biased E8M0 byte of a block: the smallest e >= -127 with 2^e * 448 >= max(amax, 1e-30),
 * taken the way the reference takes it, from the exponent and mantissa of amax. */
uint8_t oracle_mx_scale_byte(float amax) {
  if (!(amax >= 1e-30f)) {
    if (amax == amax) amax = 1e-30f; /* NaN passes through a clamp_min */
  }
  uint32_t w;
  memcpy(&w, &amax, 4);
  int biased = (int)((w >> 23) & 0xFF) - 8 + ((w & 0x7FFFFF) > 0x600000 ? 1 : 0);
  return (uint8_t)(biased < 0 ? 0 : biased);
}

/* x: bf16 bit patterns, element (r, c) at x[r*ld_row + c*ld_col]; q [rows, k] row-major
 * e4m3 bytes; scales [rows, k/32] E8M0 bytes. k must be a multiple of 32. */
void oracle_mx_quantize_bf16(const uint16_t *x, long rows, long k, long ld_row, long ld_col,
                             uint8_t *q, uint8_t *scales) {
  long blocks = k / 32;
#pragma omp parallel for schedule(static)
  for (long r = 0; r < rows; ++r) {
    for (long b = 0; b < blocks; ++b) {
      const uint16_t *src = x + r * ld_row + b * 32 * ld_col;
      float amax = 0.0f;
      int saw_nan = 0;
      for (int i = 0; i < 32; ++i) {
        float v = fabsf(bf16_to_f32(src[i * ld_col]));
        if (v != v) saw_nan = 1;
        if (v > amax) amax = v;
      }
      if (saw_nan) amax = NAN;
      uint8_t byte = oracle_mx_scale_byte(amax);
      scales[r * blocks + b] = byte;
      float inverse = ldexpf(1.0f, 127 - (int)byte);
      for (int i = 0; i < 32; ++i)
        q[r * k + b * 32 + i] = oracle_e4m3_from_f32(bf16_to_f32(src[i * ld_col]) * inverse);
    }
  }
}

/* Per-tensor recipe over n contiguous bf16 values: *scale = max(amax, 1e-12) / 448 as an
 * IEEE fp32 division, codes round x / *scale once. */
void oracle_tensor_quantize_bf16(const uint16_t *x, long n, float *scale, uint8_t *q) {
  float amax = 0.0f;
  for (long i = 0; i < n; ++i) {
    float v = fabsf(bf16_to_f32(x[i]));
    if (v > amax) amax = v;
  }
  volatile float floor_ = 1e-12f, top = 448.0f;
  float s = (amax > floor_ ? amax : floor_) / top;
  *scale = s;
#pragma omp parallel for schedule(static)
  for (long i = 0; i < n; ++i) q[i] = oracle_e4m3_from_f32(bf16_to_f32(x[i]) / s);
}
