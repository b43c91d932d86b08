// Weight-only dequant-GEMMs for gfx950: 16-bit activations times int8 / e4m3 codes that are
// widened in registers ahead of the 16-bit MFMA (V_MFMA_F32_16X16X32_{BF16,F16}).
//
//   forward   y[M,N]  = (x[M,K] @ q[N,K]^T) * scale[N] + bias[N]
//             the codes convert exactly to the activation type; scale and bias are applied to
//             the fp32 accumulator, one rounding at the store
//             (replaces the reference's Triton _fwd_kernel, backends/triton/quant.py:27-77)
//   dgrad     dx[M,K] = dy[M,N] @ W,  W[n,k] = round16(float(q[n,k]) * scale(n,k))
//             the scaled weight is rounded once to the activation type, exactly what
//             dequantize-then-matmul does (reference quant/__init__.py:26-28,43-44; Triton
//             _dgrad_kernel, backends/triton/quant.py:80-129; the 16-bit input gradient of an
//             fp8 base, backends/triton/fp8/linear.py:152-153 over fp8/formats.py:103-126).
//             scale(n,k) is one fp32 per row n, one for the tensor, one E8M0 byte per 32 codes
//             of a row (MX) or one fp32 per 128 x 128 block.
//
// One kernel template (km_wo_kernel.h): C[M,NO] = A[M,KC] @ Wd[NO,KC]^T, Wd the widened codes. A
// workgroup of four wavefronts (2 x 2) owns a BM x BN tile and walks KC in steps of 32 elements
// through a ring of four LDS stages. The A slab of a step (BM x 64 B) arrives by direct-to-LDS buffer
// loads three steps ahead. The codes come to registers four steps ahead, are widened (and scaled)
// two steps ahead and written to LDS as a 16-bit slab in the same swizzled layout, so the MFMA loop
// reads both operands alike. The MFMA operands of step s+1 are read from LDS into a second register
// set during step s: after a step's barrier the next MFMA issues at once. All of that work is cut
// into pieces of one or two instructions that ride behind single MFMAs.
//
// The forward reads the codes as they are stored, [NO, KC] with KC contiguous. The input
// gradient contracts over N, the slow axis of q[N,K]: a thread loads four consecutive k of
// eight consecutive n (eight dword loads along rows of q, each wavefront load covering whole
// 256- or 128-byte runs), transposes the 8 x 4 bytes in registers (V_PERM_B32) and widens four
// runs of eight n. No transposed copy of the frozen codes exists anywhere. Lane c of such a load
// owns columns 4c .. 4c+3, so the slab rows are stored in the order (k mod 4, k div 4) within a
// wavefront's columns, which makes every LDS write of a wavefront hit 16 consecutive rows; the
// epilogue undoes the permutation while it stages the output rows through LDS.
//
// km_wo_gemm_dgrad (with a workspace) and km_wo_gemm_dgrad_static keep the older scheme: the
// codes are first transposed to [K, N] by a small tiled kernel, then the forward's loop runs
// with a per-contraction-column scale.
//
// This file holds the entry points, the argument checks, the one-thread-per-element kernels for
// shapes the tiles do not take and the static workspace; the tile kernels are built in
// km_wo_fwd_{bf16,f16}.hip and km_wo_dgrad_{bf16,f16}.hip.
#include <hip/hip_fp16.h>
#include <stdio.h>

#include <mutex>

#include "km_gemm_common.h"
#include "km_wo_tiles.h"

namespace km {

// Any shape, any alignment: one thread per output element (the vector loads above need whole
// 16-byte chunks along the contraction axis).
template <int DT, int QF, bool DGRAD>
__global__ __launch_bounds__(256) void wo_gemm_scalar(const uint16_t* __restrict__ A, const uint8_t* __restrict__ Q,
                                                      const float* __restrict__ scale, const uint16_t* __restrict__ bias,
                                                      uint16_t* __restrict__ C, int M, int NO, int KC) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)M * NO) return;
  const int m = (int)(idx / NO), n = (int)(idx - (int64_t)m * NO);
  float acc = 0.f;
  for (int k = 0; k < KC; ++k) {
    const uint32_t byte = Q[(size_t)n * KC + k];
    float wv = QF == KM_Q_INT8 ? (float)(int)(int8_t)byte : e4m3_decode(byte);
    if (DGRAD) wv = unpack1<DT>(pack2<DT>(wv * scale[k], 0.f) & 0xFFFFu);
    acc += unpack1<DT>(A[(size_t)m * KC + k]) * wv;
  }
  if (!DGRAD) acc = acc * scale[n] + (bias ? unpack1<DT>(bias[n]) : 0.f);
  C[idx] = (uint16_t)(pack2<DT>(acc, 0.f) & 0xFFFFu);
}

// q [rows, cols] bytes -> out [cols, rows]
__global__ __launch_bounds__(256) void transpose_bytes(const uint8_t* __restrict__ in, int rows, int cols,
                                                       uint8_t* __restrict__ out) {
  __shared__ uint8_t tile[64][65];
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  for (int i = threadIdx.x; i < 64 * 64; i += 256) {
    const int r = i >> 6, c = i & 63;
    tile[r][c] = (r0 + r < rows && c0 + c < cols) ? in[(size_t)(r0 + r) * cols + c0 + c] : 0;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < 64 * 64; i += 256) {
    const int c = i >> 6, r = i & 63;
    if (r0 + r < rows && c0 + c < cols) out[(size_t)(c0 + c) * rows + r0 + r] = tile[r][c];
  }
}

struct WoConfig {
  int bm, bn, tail;
};
static const WoConfig kWoConfigs[] = {{256, 256, 0}, {128, 256, 0}, {256, 128, 0}, {128, 128, 0}, {64, 128, 0}, {256, 192, 0}, {256, 256, 1}};
static_assert(sizeof(kWoConfigs) / sizeof(kWoConfigs[0]) == kNumWoConfigs, "one row per case of launch_config");

int wo_num_configs() { return kNumWoConfigs; }
int wo_config_desc(int config, char* buf, int len) {
  if (config < 0 || config >= kNumWoConfigs) return km_fail(KM_ERR_ARG, "config out of range");
  // tail=1: half-size tiles (128 x 256 or 256 x 128) cover what whole rounds of bm x bn tiles leave over
  snprintf(buf, len, "bm=%d,bn=%d,bk=64,waves=4,tail=%d", kWoConfigs[config].bm, kWoConfigs[config].bn, kWoConfigs[config].tail);
  return KM_OK;
}

// forward, and the input gradient over a transposed copy of the codes (K-contiguous codes)
template <int DT, int QF, bool DGRAD>
static int dispatch_wo(int config, const void* a, const void* q, const float* scale, const void* bias, void* c, int M,
                       int NO, int KC, hipStream_t st) {
  // The tiles read A through a descriptor based at the tile's first row with 32-bit byte offsets: 256
  // rows of A must stay below 2^31 bytes. The forward's A is capped as a whole; the gradient dy[M, KC]
  // is not, so a very long contraction takes the element-wise kernel.
  if (!wo_tiles_take(DGRAD, a, q, KC)) {
    const int64_t n = (int64_t)M * NO;
    hipLaunchKernelGGL((wo_gemm_scalar<DT, QF, DGRAD>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                       (const uint16_t*)a, (const uint8_t*)q, scale, (const uint16_t*)bias, (uint16_t*)c, M, NO, KC);
    return km_check_launch("km_wo_gemm");
  }
  if constexpr (DGRAD) return wo_tiles_dgrad_t<DT>(QF, config, a, q, scale, c, M, NO, KC, st);
  else return wo_tiles_fwd<DT>(QF, config, a, q, scale, bias, c, M, NO, KC, st);
}

template <bool DGRAD>
static int dispatch_types(int dtype, int q_format, int config, const void* a, const void* q, const float* scale,
                          const void* bias, void* c, int M, int NO, int KC, hipStream_t st) {
  if (dtype == KM_BF16) {
    if (q_format == KM_Q_INT8) return dispatch_wo<KM_BF16, KM_Q_INT8, DGRAD>(config, a, q, scale, bias, c, M, NO, KC, st);
    return dispatch_wo<KM_BF16, KM_Q_E4M3, DGRAD>(config, a, q, scale, bias, c, M, NO, KC, st);
  }
  if (q_format == KM_Q_INT8) return dispatch_wo<KM_F16, KM_Q_INT8, DGRAD>(config, a, q, scale, bias, c, M, NO, KC, st);
  return dispatch_wo<KM_F16, KM_Q_E4M3, DGRAD>(config, a, q, scale, bias, c, M, NO, KC, st);
}

int check_wo_args(const char* who, const void* a, const void* q, const void* scale, void* c, int64_t M,
                         int64_t N, int64_t K, int q_format, int dtype, int config) {
  static thread_local char msg[160];
  const char* why = nullptr;
  if (dtype != KM_BF16 && dtype != KM_F16) why = "dtype must be bf16 or f16";
  else if (q_format != KM_Q_INT8 && q_format != KM_Q_E4M3) why = "q_format must be int8 or e4m3";
  else if (M < 0 || N < 0 || K < 0) why = "negative shape";
  else if (M * K > 0x3FFFFFFFll || N * K > 0x3FFFFFFFll || M * N > 0x7FFFFFFFFll) why = "operand too large";
  else if (config < 0 || config >= kNumWoConfigs) why = "config out of range";
  else if (M > 0 && N > 0 && K > 0 && (!a || !q || !scale || !c)) why = "null pointer";
  if (!why) return KM_OK;
  snprintf(msg, sizeof msg, "%s: %s", who, why);
  return km_fail(KM_ERR_ARG, msg);
}

// ---- the entry point that allocates nothing ----------------------------------------------------
// km_wo_gemm_dgrad_static keeps the transposed codes in this array instead of a caller's workspace.
// Every GPU the library runs on holds its own copy at its own address for the life of the process;
// host code never uses the array's name as an address, only the per-device pointer below.
constexpr int64_t kStaticCodeBytes = KM_WO_DGRAD_STATIC_MAX_CODES;
static __device__ __align__(256) uint8_t scratch[kStaticCodeBytes];
constexpr int kMaxDevices = 64;
static void* g_scratch_of_device[kMaxDevices];
static std::mutex g_scratch_lock;

// device address of `scratch` on the current device (looked up once per device)
static int static_scratch(void** out) {
  int dev = -1;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return km_fail(KM_ERR_LAUNCH, "km_wo_gemm_dgrad_static: hipGetDevice failed");
  if (dev < 0 || dev >= kMaxDevices) return km_fail(KM_ERR_UNSUPPORTED, "km_wo_gemm_dgrad_static: device index beyond 63");
  std::lock_guard<std::mutex> hold(g_scratch_lock);
  if (!g_scratch_of_device[dev]) {
    void* ptr = nullptr;
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess || !ptr) {
      static thread_local char msg[160];
      snprintf(msg, sizeof msg, "km_wo_gemm_dgrad_static: hipGetSymbolAddress: %s", hipGetErrorString(err));
      return km_fail(KM_ERR_LAUNCH, msg);
    }
    g_scratch_of_device[dev] = ptr;
  }
  *out = g_scratch_of_device[dev];
  return KM_OK;
}

}  // namespace km

using namespace km;

extern "C" int km_wo_gemm_fwd(const void* x, const void* q, const float* scale, const void* bias, void* y, int64_t M,
                              int64_t N, int64_t K, int q_format, int dtype, int config, void* stream) {
  int rc = check_wo_args("km_wo_gemm_fwd", x, q, scale, y, M, N, K, q_format, dtype, config);
  if (rc != KM_OK) return rc;
  if (M == 0 || N == 0) return KM_OK;
  return dispatch_types<false>(dtype, q_format, config, x, q, scale, bias, y, (int)M, (int)N, (int)K, (hipStream_t)stream);
}

extern "C" int km_wo_gemm_dgrad(const void* dy, const void* q, const float* scale, void* dx, void* q_t_workspace,
                                int64_t M, int64_t N, int64_t K, int q_format, int dtype, int config, void* stream) {
  int rc = check_wo_args("km_wo_gemm_dgrad", dy, q, scale, dx, M, N, K, q_format, dtype, config);
  if (rc != KM_OK) return rc;
  if (M == 0 || K == 0) return KM_OK;
  if (N > 0 && !q_t_workspace) return km_fail(KM_ERR_ARG, "km_wo_gemm_dgrad: null transpose workspace");
  hipStream_t st = (hipStream_t)stream;
  if (N > 0) {
    dim3 grid((unsigned)((K + 63) / 64), (unsigned)((N + 63) / 64));
    hipLaunchKernelGGL(transpose_bytes, grid, dim3(256), 0, st, (const uint8_t*)q, (int)N, (int)K, (uint8_t*)q_t_workspace);
  }
  // dx[M, K] = dy[M, N] @ Wd[K, N]^T with Wd = round16(q_t * scale[contraction column])
  return dispatch_types<true>(dtype, q_format, config, dy, q_t_workspace, scale, nullptr, dx, (int)M, (int)K, (int)N, st);
}

extern "C" int km_wo_gemm_dgrad_static(const void* dy, const void* q, const float* scale, void* dx, int64_t M, int64_t N,
                                       int64_t K, int q_format, int dtype, int config, void* stream) {
  // the size limit first: it is a property of the call, whatever the pointers are
  if (N > 0 && K > 0 && (N > kStaticCodeBytes || K > kStaticCodeBytes || N * K > kStaticCodeBytes)) {
    static thread_local char msg[200];
    snprintf(msg, sizeof msg, "km_wo_gemm_dgrad_static: N*K = %lld codes exceed the static workspace of %lld bytes; use km_wo_gemm_dgrad with a workspace",
             (long long)(N * K), (long long)kStaticCodeBytes);
    return km_fail(KM_ERR_UNSUPPORTED, msg);
  }
  int rc = check_wo_args("km_wo_gemm_dgrad_static", dy, q, scale, dx, M, N, K, q_format, dtype, config);
  if (rc != KM_OK) return rc;
  if (M == 0 || K == 0) return KM_OK;
  void* codes_t = nullptr;
  if (N > 0) {
    rc = static_scratch(&codes_t);
    if (rc != KM_OK) return rc;
  }
  // the transposition rewrites all N*K bytes the GEMM reads, so nothing of an earlier call shows
  return km_wo_gemm_dgrad(dy, q, scale, dx, codes_t, M, N, K, q_format, dtype, config, stream);
}

extern "C" int km_wo_gemm_path(int direction, const void* a, const void* q, const void* scale, const void* c, int64_t M, int64_t N,
                               int64_t K) {
  (void)M;
  if (direction == KM_WO_FWD) return wo_tiles_take(false, a, q, K) ? KM_PATH_TILED : KM_PATH_ELEMENTWISE;
  if (direction == KM_WO_DGRAD_W16) return wo_w16_tiles_take(a, q, scale, c, N, K) ? KM_PATH_TILED : KM_PATH_ELEMENTWISE;
  if (direction == KM_WO_DGRAD_TRANSPOSED) return wo_tiles_take(true, a, q, N) ? KM_PATH_TILED : KM_PATH_ELEMENTWISE;  // q: the transposed codes (the workspace)
  return km_fail(KM_ERR_ARG, "km_wo_gemm_path: unknown direction");
}
