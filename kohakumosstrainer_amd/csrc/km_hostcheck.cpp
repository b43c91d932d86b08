// Host build of the scalar numeric helpers (km_numeric.h) and the tile arithmetic (km_tile_plan.h) so CPU tests can check the exact
// functions the kernels use, bit by bit, against the oracle. Not part of libkm_kernels.
#include "km_numeric.h"
#include "km_tile_plan.h"

extern "C" {
unsigned km_host_e4m3_encode(float v) { return km::e4m3_encode(v); }
float km_host_e4m3_decode(unsigned code) { return km::e4m3_decode(code); }
unsigned km_host_mx_biased_exponent(float amax) { return km::mx_biased_exponent(km::f32_bits(amax) & km::kAbsMask); }
float km_host_mx_inverse_scale(unsigned biased) { return km::mx_inverse_scale(biased); }
unsigned km_host_f32_to_bf16_bits(float f) { return km::f32_to_bf16_bits(f); }
void km_host_e4m3_encode_many(const float* v, long n, unsigned char* out) {
  for (long i = 0; i < n; ++i) out[i] = (unsigned char)km::e4m3_encode(v[i]);
}
void km_host_mx_biased_many(const float* amax, long n, unsigned char* out) {
  for (long i = 0; i < n; ++i) out[i] = (unsigned char)km::mx_biased_exponent(km::f32_bits(amax[i]) & km::kAbsMask);
}
// tile of every work-group id of a tiles_m x tiles_n launch: out[2 pid] = tile_m, out[2 pid + 1] = tile_n
void km_host_tiles_of(int tiles_m, int tiles_n, int group_m, int* out) {
  for (int pid = 0; pid < tiles_m * tiles_n; ++pid) km::tile_of(pid, tiles_m, tiles_n, out[2 * pid], out[2 * pid + 1], group_m);
}
int km_host_whole_round_columns(int tiles_m, int tiles_n, int units) { return km::whole_round_columns(tiles_m, tiles_n, units); }
void km_host_bf16_many(const float* v, long n, unsigned short* out) {
  for (long i = 0; i < n; ++i) out[i] = (unsigned short)km::f32_to_bf16_bits(v[i]);
}
}
