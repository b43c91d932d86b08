// Launchers of the tiled weight-only kernels. Each activation type and direction is its own
// translation unit or several (km_wo_fwd_bf16.hip, km_wo_fwd_f16.hip, km_wo_dgrad_{bf16,f16}_{i8,e4m3,e4m3b}.hip):
// the kernels take long to compile and build side by side.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "km_internal.h"

namespace km {

constexpr int kNumWoConfigs = 7;  // 256x256, 128x256, 256x128, 128x128, 64x128, 256x192 (rows x columns of a workgroup's tile); 256x256 with a last round of half-size tiles

// y = (x @ q^T) * scale + bias over K-contiguous codes q [NO, KC]
template <int DT>
int wo_tiles_fwd(int q_format, int config, const void* a, const void* q, const float* scale, const void* bias, void* c, int M, int NO,
                 int KC, hipStream_t st);
// dx = dy @ round16(q_t^T * scale) over a transposed copy q_t [NO, KC] of the codes, scale per contraction column
template <int DT>
int wo_tiles_dgrad_t(int q_format, int config, const void* a, const void* q_t, const float* scale, void* c, int M, int NO, int KC,
                     hipStream_t st);
// dx [M, K] = dy [M, N] @ round16(q [N, K] * scale(n, k)) over the codes as stored. The kernels
// of one activation type are spread over three translation units (int8 codes; e4m3 codes with a
// scale per row or per tensor; e4m3 codes with E8M0 or 128 x 128 block scales): each `part` is
// defined in one of km_wo_dgrad_{bf16,f16}_{i8,e4m3,e4m3b}.hip.
enum { kWoPartI8 = 0, kWoPartE4m3Rows = 1, kWoPartE4m3Blocks = 2 };
template <int DT, int PART>
int wo_tiles_dgrad_n_part(int scale_kind, int config, const void* dy, const void* q, const void* scale, int scale_ld, void* dx, int M,
                          int N, int K, hipStream_t st);
template <int DT>
inline int wo_tiles_dgrad_n(int q_format, int scale_kind, int config, const void* dy, const void* q, const void* scale, int scale_ld,
                            void* dx, int M, int N, int K, hipStream_t st) {
  if (q_format == KM_Q_INT8) return wo_tiles_dgrad_n_part<DT, kWoPartI8>(scale_kind, config, dy, q, scale, scale_ld, dx, M, N, K, st);
  if (scale_kind == KM_WSCALE_ROWS) return wo_tiles_dgrad_n_part<DT, kWoPartE4m3Rows>(scale_kind, config, dy, q, scale, scale_ld, dx, M, N, K, st);
  return wo_tiles_dgrad_n_part<DT, kWoPartE4m3Blocks>(scale_kind, config, dy, q, scale, scale_ld, dx, M, N, K, st);
}

// longest row of a 16-bit operand that a 256-row tile can address with 32-bit byte offsets
constexpr int kMaxTiledRowElems = 0x7FFFFFFF / (256 * 2);

// Whether a problem runs on the tiled kernels; anything else goes to a kernel with one thread per output
// element, which is correct for every shape and alignment and far slower. The dispatchers and
// km_wo_gemm_path() ask the same functions.
// forward / input gradient over transposed codes: A [M, KC] 16-bit, codes [NO, KC]
inline bool wo_tiles_take(bool dgrad, const void* a, const void* q, int64_t KC) {
  return KC % 8 == 0 && !(dgrad && KC > kMaxTiledRowElems) && ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(q)) & 15) == 0;
}
// input gradient over the codes as stored: dy [M, N], q [N, K], dx [M, K]. An empty contraction takes
// the element-wise kernel too (it writes zeros and reads no operand); so does a q so wide that 32 of its
// rows pass 2^31 bytes (the tiled kernels step through q by that stride), and a contraction so long that
// the 256 rows of dy a tile reads pass 2^31 bytes (32-bit offsets from the tile's first row)
inline bool wo_w16_tiles_take(const void* dy, const void* q, const void* scale, const void* dx, int64_t N, int64_t K) {
  const uintptr_t bits = reinterpret_cast<uintptr_t>(dy) | reinterpret_cast<uintptr_t>(dx);
  return N != 0 && N % 8 == 0 && K % 4 == 0 && K <= 0x7FFFFFFF / 32 && N <= kMaxTiledRowElems && (bits & 15) == 0 &&
         (reinterpret_cast<uintptr_t>(q) & 3) == 0 && (reinterpret_cast<uintptr_t>(scale) & 3) == 0;
}

// argument checks shared by the entry points
int check_wo_args(const char* who, const void* a, const void* q, const void* scale, void* c, int64_t M, int64_t N, int64_t K,
                  int q_format, int dtype, int config);

}  // namespace km
