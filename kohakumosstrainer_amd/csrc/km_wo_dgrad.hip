// Input gradient of int8 / e4m3 weight-only bases and of fp8 compute bases without a transposed
// copy, over the codes as they are stored: dx[M,K] = dy[M,N] @ round16(q[N,K] * scale(n,k)). The
// tiled kernel (km_wo_kernel.h, mode kWoDgradN; built in km_wo_dgrad_{bf16,f16}_{i8,e4m3,e4m3b}.hip) transposes 8 x 4 bytes of codes in registers on
// their way to LDS; shapes it does not take go to a one-thread-per-element kernel.
#include "km_gemm_common.h"
#include "km_wo_tiles.h"

namespace km {

// the scale of code (n, k) of q[N, K] for the three layouts of the input gradient
template <int SK>
__device__ __forceinline__ float weight_scale(const void* scale, int64_t ld, int n, int k) {
  if constexpr (SK == KM_WSCALE_ROWS) return static_cast<const float*>(scale)[n * ld];
  else if constexpr (SK == KM_WSCALE_E8M0) return bits_f32((uint32_t)static_cast<const uint8_t*>(scale)[n * ld + (k >> 5)] << 23);
  else return static_cast<const float*>(scale)[(n >> 7) * ld + (k >> 7)];
}

// dx[m, k] = sum_n dy[m, n] * round16(q[n, k] * scale(n, k)) for shapes the tiled kernel does not take
template <int DT, int QF, int SK>
__global__ __launch_bounds__(256) void wo_dgrad_scalar(const uint16_t* __restrict__ dy, const uint8_t* __restrict__ Q,
                                                       const void* __restrict__ scale, int scale_ld, uint16_t* __restrict__ dx,
                                                       int M, int N, int K) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)M * K) return;
  const int m = (int)(idx / K), k = (int)(idx - (int64_t)m * K);
  float acc = 0.f;
  for (int n = 0; n < N; ++n) {
    const uint32_t byte = Q[(size_t)n * K + k];
    const float code = QF == KM_Q_INT8 ? (float)(int)(int8_t)byte : e4m3_decode(byte);
    const float wv = unpack1<DT>(pack2<DT>(code * weight_scale<SK>(scale, scale_ld, n, k), 0.f) & 0xFFFFu);
    acc += unpack1<DT>(dy[(size_t)m * N + n]) * wv;
  }
  dx[idx] = (uint16_t)(pack2<DT>(acc, 0.f) & 0xFFFFu);
}

// the input gradient over q as stored: dx[M, K] = dy[M, N] @ round16(q[N, K] * scale)
template <int DT, int QF, int SK>
static int dispatch_w16(int config, const void* dy, const void* q, const void* scale, int scale_ld, void* dx, int M, int N,
                        int K, hipStream_t st) {
  if (!wo_w16_tiles_take(dy, q, scale, dx, N, K)) {
    const int64_t n = (int64_t)M * K;
    hipLaunchKernelGGL((wo_dgrad_scalar<DT, QF, SK>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, (const uint16_t*)dy,
                       (const uint8_t*)q, scale, scale_ld, (uint16_t*)dx, M, N, K);
    return km_check_launch("km_wo_gemm_dgrad_w16");
  }
  return wo_tiles_dgrad_n<DT>(QF, SK, config, dy, q, scale, scale_ld, dx, M, N, K, st);
}

template <int DT>
static int dispatch_w16_formats(int q_format, int scale_kind, int config, const void* dy, const void* q, const void* scale,
                                int scale_ld, void* dx, int M, int N, int K, hipStream_t st) {
  if (q_format == KM_Q_INT8) return dispatch_w16<DT, KM_Q_INT8, KM_WSCALE_ROWS>(config, dy, q, scale, scale_ld, dx, M, N, K, st);
  if (scale_kind == KM_WSCALE_ROWS) return dispatch_w16<DT, KM_Q_E4M3, KM_WSCALE_ROWS>(config, dy, q, scale, scale_ld, dx, M, N, K, st);
  if (scale_kind == KM_WSCALE_E8M0) return dispatch_w16<DT, KM_Q_E4M3, KM_WSCALE_E8M0>(config, dy, q, scale, scale_ld, dx, M, N, K, st);
  return dispatch_w16<DT, KM_Q_E4M3, KM_WSCALE_BLOCKS>(config, dy, q, scale, scale_ld, dx, M, N, K, st);
}

}  // namespace km

using namespace km;

extern "C" int km_wo_gemm_dgrad_w16(const void* dy, const void* q, const void* scale, int scale_kind, int64_t scale_ld, void* dx,
                                    int64_t M, int64_t N, int64_t K, int q_format, int dtype, int config, void* stream) {
  int rc = check_wo_args("km_wo_gemm_dgrad_w16", dy, q, scale, dx, M, N, K, q_format, dtype, config);
  if (rc != KM_OK) return rc;
  static thread_local char msg[200];
  const char* why = nullptr;
  if (scale_kind != KM_WSCALE_ROWS && scale_kind != KM_WSCALE_E8M0 && scale_kind != KM_WSCALE_BLOCKS) why = "unknown scale_kind";
  else if (q_format == KM_Q_INT8 && scale_kind != KM_WSCALE_ROWS) why = "int8 codes take one scale per row";
  else if (scale_kind == KM_WSCALE_ROWS && scale_ld != 0 && scale_ld != 1) why = "scale_ld of row scales is 1, or 0 for one scale of the whole tensor";
  else if (scale_kind == KM_WSCALE_E8M0 && scale_ld < (K + 31) / 32) why = "scale_ld of E8M0 scales is at least ceil(K / 32)";
  else if (scale_kind == KM_WSCALE_BLOCKS && scale_ld < (K + 127) / 128) why = "scale_ld of 128 x 128 block scales is at least ceil(K / 128)";
  else if (scale_ld > 0x7FFFFFFF || N * scale_ld > 0x7FFFFFFFll) why = "scale operand too large";
  if (why) {
    snprintf(msg, sizeof msg, "km_wo_gemm_dgrad_w16: %s", why);
    return km_fail(KM_ERR_ARG, msg);
  }
  if (M == 0 || K == 0) return KM_OK;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == KM_BF16)
    return dispatch_w16_formats<KM_BF16>(q_format, scale_kind, config, dy, q, scale, (int)scale_ld, dx, (int)M, (int)N, (int)K, st);
  return dispatch_w16_formats<KM_F16>(q_format, scale_kind, config, dy, q, scale, (int)scale_ld, dx, (int)M, (int)N, (int)K, st);
}

