// Weight-only dequant-GEMMs for gfx950: 16-bit activations times int8 / e4m3 codes that are
// widened in registers ahead of the 16-bit MFMA (V_MFMA_F32_16X16X32_{BF16,F16}).
//
//   forward   y[M,N]  = (x[M,K] @ q[N,K]^T) * scale[N] + bias[N]
//             the codes convert exactly to the activation type; scale and bias are applied to
//             the fp32 accumulator, one rounding at the store
//             (replaces the reference's Triton _fwd_kernel, backends/triton/quant.py:27-77)
//   dgrad     dx[M,K] = dy[M,N] @ W,  W[n,k] = round16(float(q[n,k]) * scale[n])
//             the scaled weight is rounded once to the activation type, exactly what
//             dequantize-then-matmul does (reference quant/__init__.py:26-28,43-44; Triton
//             _dgrad_kernel, backends/triton/quant.py:80-129). The contraction runs over N, so
//             the codes are first transposed to [K, N] by a small tiled kernel.
//
// Both are one kernel: C[M,NO] = A[M,KC] @ Wd[NO,KC]^T with Wd = widen(codes[NO,KC]) and either
// a per-output-column scale in the epilogue (forward) or a per-contraction-column scale before
// the rounding (dgrad). A workgroup of four wavefronts (2 x 2) owns a BM x BN tile and walks KC
// in steps of 64 elements. The A slab (BM x 128 B) arrives by direct-to-LDS buffer loads; the
// codes (BN x 64 B) are loaded to registers, widened (and scaled) there and written to LDS as a
// 16-bit slab in the same swizzled layout, so the MFMA loop reads both operands alike. Two
// stages, one barrier per step; the global loads of step k+1 are issued between the MFMAs of
// step k.
#include <hip/hip_fp16.h>
#include <stdio.h>

#include <mutex>

#include "km_gemm_common.h"

namespace km {

typedef short v8s __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

constexpr int kWoStepElems = 64;  // contraction elements per step (128 B of 16-bit values)

template <int DT>
__device__ __forceinline__ void mfma16(v4f& c, const v4i& a, const v4i& b) {
  if constexpr (DT == KM_BF16)
    asm("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  else
    asm("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}

// 8 codes (two dwords) -> 8 values of the activation type (four dwords); `s` scales them in
// fp32 before the single rounding (dgrad), or is 1 (forward: the conversion is exact)
typedef float v2f __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));

// four e4m3 codes of one dword -> four fp32 (V_CVT_PK_F32_FP8, two codes per instruction)
__device__ __forceinline__ void e4m3x4_to_f32(uint32_t w, float (&f)[4]) {
  const v2f lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false), hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
  f[0] = lo.x; f[1] = lo.y; f[2] = hi.x; f[3] = hi.y;
}
// four e4m3 codes -> two dwords of the activation type: every e4m3 value is exact in bf16 and
// f16, so the scaled conversion with scale 1 is the whole job (two codes per instruction)
template <int DT>
__device__ __forceinline__ uint2 e4m3x4_to_16(uint32_t w) {
  if constexpr (DT == KM_BF16)
    return make_uint2(__builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false)),
                      __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true)));
  else
    return make_uint2(__builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, false)),
                      __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, true)));
}

template <int DT, int QF, bool SCALE>
__device__ __forceinline__ uint4 widen_codes(uint2 raw, const float (&s)[8]) {
  if constexpr (QF == KM_Q_E4M3 && !SCALE) {
    const uint2 lo = e4m3x4_to_16<DT>(raw.x), hi = e4m3x4_to_16<DT>(raw.y);
    return make_uint4(lo.x, lo.y, hi.x, hi.y);
  } else {
    float f[8];
    if constexpr (QF == KM_Q_E4M3) {
      float a[4], b[4];
      e4m3x4_to_f32(raw.x, a);
      e4m3x4_to_f32(raw.y, b);
#pragma unroll
      for (int i = 0; i < 4; ++i) { f[i] = a[i]; f[4 + i] = b[i]; }
    } else {
      const uint32_t w[2] = {raw.x, raw.y};
#pragma unroll
      for (int i = 0; i < 8; ++i) f[i] = (float)(int)(int8_t)((w[i >> 2] >> (8 * (i & 3))) & 0xFFu);
    }
    if constexpr (SCALE) {
#pragma unroll
      for (int i = 0; i < 8; ++i) f[i] *= s[i];
    }
    return make_uint4(pack2<DT>(f[0], f[1]), pack2<DT>(f[2], f[3]), pack2<DT>(f[4], f[5]), pack2<DT>(f[6], f[7]));
  }
}

template <int BM, int BN, int DT, int QF, bool DGRAD>
__global__ __launch_bounds__(256) void wo_gemm_kernel(const uint16_t* __restrict__ A, const uint8_t* __restrict__ Q,
                                                      const float* __restrict__ scale, const uint16_t* __restrict__ bias,
                                                      uint16_t* __restrict__ C, int M, int NO, int KC) {
  constexpr int WTM = BM / 2, WTN = BN / 2;
  constexpr int TM = WTM / 16, TN = WTN / 16;
  constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128;
  constexpr int A_LD = BM / 32;   // direct-to-LDS passes of 32 rows per step
  constexpr int Q_LD = BN / 32;   // 8-byte code loads per thread per step (32 rows x 8 lanes per pass)
  __shared__ __attribute__((aligned(1024))) uint8_t a_buf0[A_BYTES];
  __shared__ __attribute__((aligned(1024))) uint8_t a_buf1[A_BYTES];
  __shared__ __attribute__((aligned(1024))) uint8_t b_buf0[B_BYTES];
  __shared__ __attribute__((aligned(1024))) uint8_t b_buf1[B_BYTES];

  int tile_m, tile_n;
  tile_of(blockIdx.x, (M + BM - 1) / BM, (NO + BN - 1) / BN, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = (wave >> 1) * WTM, wn = (wave & 1) * WTN;
  const int r16 = lane & 15, g = lane >> 4;
  const int nk = (KC + kWoStepElems - 1) / kWoStepElems;

  const v4i a_rsrc = raw_rsrc(A + (size_t)m0 * KC, (uint32_t)min((int64_t)(M - m0) * KC * 2, (int64_t)0x7FFFFFFF));
  const __amdgpu_buffer_rsrc_t q_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t*>(Q) + (size_t)n0 * KC, 0, (int)min((int64_t)(NO - n0) * KC, (int64_t)0x7FFFFFFF), 0x00020000);
  // staging map of a pass: 8 lanes per row; 16 lanes cover rows r and r+8 (one LDS line)
  const int w = tid >> 3;
  const int srow = ((w >> 4) << 4) + ((w & 1) << 3) + ((w >> 1) & 7);  // 0 .. 31
  const int a_chunk = (tid & 7) ^ (srow & 7);  // the direct-to-LDS load lands in slot tid & 7
  const int q_chunk = tid & 7;                 // the register path writes slab_offset() itself
  constexpr int kOob = 0x7FFFFFFF;             // an offset past every buffer: the load returns 0

  v4f acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

  uint2 qraw[Q_LD];
  float qscale[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) qscale[i] = 1.f;

  // Columns past KC are turned into out-of-range offsets (whole 8-element chunks, KC % 8 == 0),
  // rows past the end are out of range by themselves: both read as zeros.
  auto dma_a_pass = [&](uint8_t* buf, int ks, int i) __attribute__((always_inline)) {
    const int col = ks * kWoStepElems + a_chunk * 8;
    const int voff = col < KC ? ((srow + i * 32) * KC + col) * 2 : kOob;
    hidden_dma_b128(a_rsrc, lds_offset(buf) + i * 4096 + wave * 1024, voff, 0);  // waited for at the end of the step
  };
  auto q_load_pass = [&](int ks, int i) __attribute__((always_inline)) {
    const int col = ks * kWoStepElems + q_chunk * 8;
    const int voff = col < KC ? (srow + i * 32) * KC + col : kOob;
    qraw[i] = __builtin_bit_cast(uint2, __builtin_amdgcn_raw_buffer_load_b64(q_rsrc, voff, 0, 0));
  };
  auto q_scale_load = [&](int ks) __attribute__((always_inline)) {
    if constexpr (DGRAD) {
      const int col = ks * kWoStepElems + q_chunk * 8;  // whole chunks: KC % 8 == 0
      float4 lo = make_float4(0.f, 0.f, 0.f, 0.f), hi = lo;
      if (col < KC) {
        lo = *reinterpret_cast<const float4*>(scale + col);
        hi = *reinterpret_cast<const float4*>(scale + col + 4);
      }
      qscale[0] = lo.x; qscale[1] = lo.y; qscale[2] = lo.z; qscale[3] = lo.w;
      qscale[4] = hi.x; qscale[5] = hi.y; qscale[6] = hi.z; qscale[7] = hi.w;
    }
  };
  auto q_commit = [&](uint8_t* buf) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < Q_LD; ++i)
      *reinterpret_cast<uint4*>(buf + slab_offset(srow + i * 32, q_chunk)) = widen_codes<DT, QF, DGRAD>(qraw[i], qscale);
  };
  auto fragment = [&](const uint8_t* slab, int row, int sub) __attribute__((always_inline)) -> v4i {
    return *reinterpret_cast<const v4i*>(slab + slab_offset(row, 4 * sub + g));
  };

  // One step: fetch step ks+1 (A by direct-to-LDS, codes to registers) between the MFMAs of
  // step ks, then widen the codes into the other B buffer and pass the barrier.
  constexpr int kSlots = 2 * TN * TM;  // MFMAs per step
  auto step = [&](const uint8_t* a_cur, uint8_t* a_nxt, const uint8_t* b_cur, uint8_t* b_nxt, int ks)
                  __attribute__((always_inline)) {
    const int next = ks + 1;  // may be nk: every column is out of range then, the loads return 0
    static_for<2>([&](auto s_tag) __attribute__((always_inline)) {
      constexpr int sub = decltype(s_tag)::value;
      v4i xf[TM];
#pragma unroll
      for (int j = 0; j < TM; ++j) xf[j] = fragment(a_cur, wm + j * 16 + r16, sub);
      static_for<TN>([&](auto t_tag) __attribute__((always_inline)) {
        constexpr int t = decltype(t_tag)::value;
        const v4i wf = fragment(b_cur, wn + t * 16 + r16, sub);
        static_for<TM>([&](auto j_tag) __attribute__((always_inline)) {
          constexpr int j = decltype(j_tag)::value;
          constexpr int q = (sub * TN + t) * TM + j;
          mfma16<DT>(acc[t][j], wf, xf[j]);
          static_for<Q_LD>([&](auto i_tag) __attribute__((always_inline)) {
            constexpr int i = decltype(i_tag)::value;
            if constexpr (q == i * (kSlots / 4) / Q_LD) q_load_pass(next, i);
          });
          static_for<A_LD>([&](auto i_tag) __attribute__((always_inline)) {
            constexpr int i = decltype(i_tag)::value;
            if constexpr (q == kSlots / 4 + i * (kSlots / 2) / A_LD) dma_a_pass(a_nxt, next, i);
          });
        });
      });
    });
    q_commit(b_nxt);
    q_scale_load(next + 1);
    __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(DGRAD ? 2 : 0));  // all but the two newest (scale) loads
    __syncthreads();
  };

  // prologue
#pragma unroll
  for (int i = 0; i < A_LD; ++i) dma_a_pass(a_buf0, 0, i);
  q_scale_load(0);
#pragma unroll
  for (int i = 0; i < Q_LD; ++i) q_load_pass(0, i);
  __builtin_amdgcn_s_waitcnt(kWaitVm0);
  q_commit(b_buf0);
  q_scale_load(1);
  __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(DGRAD ? 2 : 0));
  __syncthreads();

  for (int ks = 0; ks < nk; ks += 2) {
    step(a_buf0, a_buf1, b_buf0, b_buf1, ks);
    if (ks + 1 < nk) step(a_buf1, a_buf0, b_buf1, b_buf0, ks + 1);
  }
  __builtin_amdgcn_s_waitcnt(kWaitVm0);
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);

  if constexpr (DGRAD)
    store_tile<BM, BN, DT, 0>(acc, 1.0f, nullptr, nullptr, nullptr, C, M, NO, m0, n0, a_buf0, a_buf1, b_buf0, b_buf1);
  else
    store_tile<BM, BN, DT, 1>(acc, 1.0f, nullptr, scale, bias, C, M, NO, m0, n0, a_buf0, a_buf1, b_buf0, b_buf1);
}

// Any shape, any alignment: one thread per output element (contraction lengths that are not a
// multiple of 8 cannot take the vector loads above).
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
  int bm, bn;
};
static const WoConfig kWoConfigs[] = {{256, 256}, {128, 256}, {256, 128}, {128, 128}, {64, 128}};
constexpr int kNumWoConfigs = sizeof(kWoConfigs) / sizeof(kWoConfigs[0]);

int wo_num_configs() { return kNumWoConfigs; }
int wo_config_desc(int config, char* buf, int len) {
  if (config < 0 || config >= kNumWoConfigs) return km_fail(KM_ERR_ARG, "config out of range");
  snprintf(buf, len, "bm=%d,bn=%d,bk=64,waves=4", kWoConfigs[config].bm, kWoConfigs[config].bn);
  return KM_OK;
}

template <int BM, int BN, int DT, int QF, bool DGRAD>
static int launch_wo(const void* a, const void* q, const float* scale, const void* bias, void* c, int M, int NO, int KC,
                     hipStream_t st) {
  const int tiles = ((M + BM - 1) / BM) * ((NO + BN - 1) / BN);
  hipLaunchKernelGGL((wo_gemm_kernel<BM, BN, DT, QF, DGRAD>), dim3(tiles), dim3(256), 0, st, (const uint16_t*)a,
                     (const uint8_t*)q, scale, (const uint16_t*)bias, (uint16_t*)c, M, NO, KC);
  return km_check_launch("km_wo_gemm");
}

template <int DT, int QF, bool DGRAD>
static int dispatch_wo(int config, const void* a, const void* q, const float* scale, const void* bias, void* c, int M,
                       int NO, int KC, hipStream_t st) {
  if (KC % 8 || ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(q)) & 15)) {
    const int64_t n = (int64_t)M * NO;
    hipLaunchKernelGGL((wo_gemm_scalar<DT, QF, DGRAD>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                       (const uint16_t*)a, (const uint8_t*)q, scale, (const uint16_t*)bias, (uint16_t*)c, M, NO, KC);
    return km_check_launch("km_wo_gemm");
  }
  switch (config) {
    case 0: return launch_wo<256, 256, DT, QF, DGRAD>(a, q, scale, bias, c, M, NO, KC, st);
    case 1: return launch_wo<128, 256, DT, QF, DGRAD>(a, q, scale, bias, c, M, NO, KC, st);
    case 2: return launch_wo<256, 128, DT, QF, DGRAD>(a, q, scale, bias, c, M, NO, KC, st);
    case 3: return launch_wo<128, 128, DT, QF, DGRAD>(a, q, scale, bias, c, M, NO, KC, st);
    case 4: return launch_wo<64, 128, DT, QF, DGRAD>(a, q, scale, bias, c, M, NO, KC, st);
  }
  return km_fail(KM_ERR_ARG, "km_wo_gemm: unknown config");
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

static int check_wo_args(const char* who, const void* a, const void* q, const float* scale, void* c, int64_t M,
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
