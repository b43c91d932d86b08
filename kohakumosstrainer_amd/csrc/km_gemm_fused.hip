// One-launch fp8 linears for short M on gfx950: C = Q(x) B^T (+ bias) with x [M,K] bf16 / fp16
// quantized inside the K loop and B [N,K] e4m3 quantized beforehand, in three recipes:
//
//   mx     E8M0 exponent per 32 columns, e4m3 codes (the arithmetic of the row-wise MX quantizer
//          kernel, so the codes are the ones km_quant_mx writes); B comes with its MFMA-packed
//          E8M0 scales and the block-scaled MFMA applies both
//   row    one fp32 scale per token row (a prologue scans the rows for their abs-max), unit MFMA
//          scales, s[m] * wscale[n] on the sum at the end
//   block  one fp32 scale per row and 128 columns: a K step is one block, its MFMA sum starts from
//          zero and is promoted with s[m, kb] * wscale[n / 128, kb]
//
// Replaces the reference's Triton fused kernels (src/kohakumoss_kernels/backends/triton/fp8/fused.py:
// _fused_mx_kernel :98-120, _fused_row_kernel :35-68, _fused_block_kernel :71-95): at M <= 256 the
// reference's linear is bound by launches, not by the MMA, and one launch replaces two.
//
// Shape of the kernel. At short M the job is to stream the weight once, so there is no LDS
// staging and no barrier in the K loop: a workgroup owns 16*TM tokens x 64 output columns (32 when
// N is not a multiple of 64) and its WAVES wavefronts split K (wavefront w takes K steps w,
// w + WAVES, ...), each loading its MFMA fragments straight from global memory in the MFMA's own
// layout (lane l: row l%16, K bytes [16g, 16g+16) and [64+16g, 64+16g+16) with g = l/16), one to
// three steps ahead in registers. N/64 workgroups (144 at N = 9216) stream the weight; every one
// of them quantizes its rows of x again, which is what bounds the useful M. For mx, a 32-column
// block of x lies in two lanes (g and g^1): they share their 16-bit abs-max with one cross-lane
// exchange, and a second one hands each lane the exponent byte the MFMA expects from it (lane g
// supplies block g). The partial sums of a workgroup meet in LDS at the end.
#include <stdio.h>

#include "km_gemm_common.h"
#include "km_quant_common.h"

namespace km {

constexpr int kFusedBN = 32;
constexpr int kFusedMaxTM = 4;

// The quantizer kernels convert with MODE.FP16_OVFL set (out-of-range values saturate at +-448).
// Here the mode stays clear, because the same wavefront's MFMAs would read the e4m3 NaN codes as
// numbers under it. A finite block never leaves the e4m3 range (its exponent is chosen so that
// amax * 2^-e <= 448), so only the non-finite inputs themselves need the codes the saturating
// conversion and the reference give them: infinity -> +-448 (0x7E), NaN -> 0x7F, sign kept.
template <int DT>
__device__ __forceinline__ uint32_t nonfinite_fix(uint32_t codes, uint32_t h, int shift) {
  const uint32_t a0 = h & 0x7FFFu, a1 = (h >> 16) & 0x7FFFu;
  if (a0 >= inf16<DT>()) codes = (codes & ~(0xFFu << shift)) | (((a0 > inf16<DT>() ? 0x7Fu : 0x7Eu) | ((h >> 8) & 0x80u)) << shift);
  if (a1 >= inf16<DT>()) codes = (codes & ~(0xFF00u << shift)) | (((a1 > inf16<DT>() ? 0x7Fu : 0x7Eu) | ((h >> 24) & 0x80u)) << (shift + 8));
  return codes;
}

constexpr int kFusedMx = 0, kFusedRow = 1, kFusedBlock = 2;

// WAVES wavefronts split K (4, or 8 for a single row tile: three K steps each at K = 3072, all of
// them in flight at once).
template <int DT, int OUT, int TM, int TN, int MODE, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void gemm_mx_fused_kernel(const uint16_t* __restrict__ X, int64_t ldx, const uint8_t* __restrict__ B,
                                                            const uint8_t* __restrict__ Bs, const float* __restrict__ wscales,
                                                            const uint16_t* __restrict__ bias, uint16_t* __restrict__ C, int M, int N, int K) {
  constexpr bool ROW = MODE == kFusedRow, BLOCK = MODE == kFusedBlock;
  constexpr int BN = 16 * TN;  // 32 output columns, or 64: half as many workgroups quantize x again
  __shared__ float4 partial[WAVES][TM * TN][64];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r16 = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * BN, m0 = blockIdx.y * (16 * TM);
  const int nk = K / kStepBytes;
  const int row_groups = (N + 127) >> 7;

  struct Slab {
    uint4 a[TM][4];   // x: elements [16g, 16g+8), [16g+8, 16g+16), [64+16g, +8), [64+16g+8, +8)
    uint4 b[TN][2];   // codes: bytes [16g, 16g+16), [64+16g, 64+16g+16)
    uint2 bs;         // mx: packed scale bytes of the eight 16-row tiles of this row group, block g
    float wb;         // block recipe: the scale of this step's 128 x 128 weight block
  };
  auto load = [&](Slab& s, int ks) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      const int m = m0 + j * 16 + r16;
      const uint4* p = reinterpret_cast<const uint4*>(X + (int64_t)m * ldx + ks * kStepBytes + 16 * g);
      const bool live = m < M;
      s.a[j][0] = live ? p[0] : make_uint4(0, 0, 0, 0);
      s.a[j][1] = live ? p[1] : make_uint4(0, 0, 0, 0);
      s.a[j][2] = live ? p[8] : make_uint4(0, 0, 0, 0);
      s.a[j][3] = live ? p[9] : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int t = 0; t < TN; ++t) {
      const uint4* p = reinterpret_cast<const uint4*>(B + (int64_t)(n0 + t * 16 + r16) * K + ks * kStepBytes + 16 * g);
      s.b[t][0] = p[0];
      s.b[t][1] = p[4];
    }
    if constexpr (MODE == kFusedMx) s.bs = *reinterpret_cast<const uint2*>(Bs + (((int64_t)ks * row_groups + (n0 >> 7)) * 16 + r16) * 32 + 8 * g);
    if constexpr (BLOCK) s.wb = wscales[(int64_t)(n0 >> 7) * nk + ks];
  };

  // ROW: scale, its rounded reciprocal and the kind of every token row of this lane (row j * 16 + r16)
  float s_row[TM], r_row[TM];
  bool finite_row[TM], nan_row[TM];
  if constexpr (ROW) {
    __shared__ uint32_t row_amax[WAVES][TM][16];
    uint32_t m16[TM];
#pragma unroll
    for (int j = 0; j < TM; ++j) m16[j] = 0;
    for (int ks = wave; ks < nk; ks += WAVES) {
#pragma unroll
      for (int j = 0; j < TM; ++j) {
        const int m = m0 + j * 16 + r16;
        if (m < M) {
          const uint4* p = reinterpret_cast<const uint4*>(X + (int64_t)m * ldx + ks * kStepBytes + 16 * g);
          const uint32_t a0 = amax16x8(p[0]), a1 = amax16x8(p[1]), a2 = amax16x8(p[8]), a3 = amax16x8(p[9]);
          const uint32_t a01 = a0 > a1 ? a0 : a1, a23 = a2 > a3 ? a2 : a3, a = a01 > a23 ? a01 : a23;
          m16[j] = a > m16[j] ? a : m16[j];
        }
      }
    }
#pragma unroll
    for (int j = 0; j < TM; ++j) {  // the four lanes (g) that share a row, then the four wavefronts
      uint32_t o = (uint32_t)__shfl_xor((int)m16[j], 16);
      m16[j] = o > m16[j] ? o : m16[j];
      o = (uint32_t)__shfl_xor((int)m16[j], 32);
      m16[j] = o > m16[j] ? o : m16[j];
      if (g == 0) row_amax[wave][j][r16] = m16[j];
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      uint32_t mm = row_amax[0][j][r16];
#pragma unroll
      for (int w = 1; w < WAVES; ++w) mm = max(mm, row_amax[w][j][r16]);
      s_row[j] = scale_of_amax16<DT>(mm);
      r_row[j] = __fdiv_rn(1.0f, s_row[j]);
      finite_row[j] = mm < inf16<DT>();
      nan_row[j] = mm > inf16<DT>();
    }
  }

  v4f acc[TN][TM];
#pragma unroll
  for (int t = 0; t < TN; ++t)
#pragma unroll
    for (int j = 0; j < TM; ++j) acc[t][j] = v4f{0.f, 0.f, 0.f, 0.f};

  auto compute = [&](const Slab& s) __attribute__((always_inline)) {
    uint64_t bs64 = 0x7F7F7F7F7F7F7F7Full;  // row and block recipes: unit MFMA scales
    if constexpr (MODE == kFusedMx) bs64 = ((uint64_t)s.bs.y << 32 | s.bs.x) >> (((n0 & 127) >> 4) * 8);
    v8i wf[TN];
    int wscale[TN];
#pragma unroll
    for (int t = 0; t < TN; ++t) {
      wf[t] = v8i{(int)s.b[t][0].x, (int)s.b[t][0].y, (int)s.b[t][0].z, (int)s.b[t][0].w, (int)s.b[t][1].x, (int)s.b[t][1].y, (int)s.b[t][1].z, (int)s.b[t][1].w};
      wscale[t] = (int)((bs64 >> (8 * t)) & 0xFFu);
    }
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      if constexpr (BLOCK) {
        const uint32_t a0 = amax16x8(s.a[j][0]), a1 = amax16x8(s.a[j][1]), a2 = amax16x8(s.a[j][2]), a3 = amax16x8(s.a[j][3]);
        const uint32_t a01 = a0 > a1 ? a0 : a1, a23 = a2 > a3 ? a2 : a3;
        uint32_t mm = a01 > a23 ? a01 : a23;
        uint32_t o = (uint32_t)__shfl_xor((int)mm, 16);
        mm = o > mm ? o : mm;
        o = (uint32_t)__shfl_xor((int)mm, 32);
        mm = o > mm ? o : mm;
        const float sc = scale_of_amax16<DT>(mm), rc = __fdiv_rn(1.0f, sc);
        const bool fin = mm < inf16<DT>(), nan = mm > inf16<DT>();
        const uint2 c0 = divided_codes8<DT>(s.a[j][0], sc, rc, fin, nan), c1 = divided_codes8<DT>(s.a[j][1], sc, rc, fin, nan);
        const uint2 c2 = divided_codes8<DT>(s.a[j][2], sc, rc, fin, nan), c3 = divided_codes8<DT>(s.a[j][3], sc, rc, fin, nan);
        const v8i xf = v8i{(int)c0.x, (int)c0.y, (int)c1.x, (int)c1.y, (int)c2.x, (int)c2.y, (int)c3.x, (int)c3.y};
        const float promote = sc * s.wb;
#pragma unroll
        for (int t = 0; t < TN; ++t) {
          const v4f part = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[t], xf, v4f{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0x7F, 0, 0x7F);
#pragma unroll
          for (int v = 0; v < 4; ++v) acc[t][j][v] = __builtin_fmaf(part[v], promote, acc[t][j][v]);
        }
        continue;
      }
      if constexpr (ROW) {
        const uint2 c0 = divided_codes8<DT>(s.a[j][0], s_row[j], r_row[j], finite_row[j], nan_row[j]);
        const uint2 c1 = divided_codes8<DT>(s.a[j][1], s_row[j], r_row[j], finite_row[j], nan_row[j]);
        const uint2 c2 = divided_codes8<DT>(s.a[j][2], s_row[j], r_row[j], finite_row[j], nan_row[j]);
        const uint2 c3 = divided_codes8<DT>(s.a[j][3], s_row[j], r_row[j], finite_row[j], nan_row[j]);
        const v8i xf = v8i{(int)c0.x, (int)c0.y, (int)c1.x, (int)c1.y, (int)c2.x, (int)c2.y, (int)c3.x, (int)c3.y};
#pragma unroll
        for (int t = 0; t < TN; ++t)
          acc[t][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[t], xf, acc[t][j], 0, 0, 0, 0x7F, 0, 0x7F);
        continue;
      }
      // abs-max of this lane's two 16-element halves, then of the 32-column blocks they belong to
      const uint32_t a0 = amax16x8(s.a[j][0]), a1 = amax16x8(s.a[j][1]), a2 = amax16x8(s.a[j][2]), a3 = amax16x8(s.a[j][3]);
      uint32_t m_lo = a0 > a1 ? a0 : a1, m_hi = a2 > a3 ? a2 : a3;
      const uint32_t other = (uint32_t)__shfl_xor((int)(m_lo | (m_hi << 16)), 16);
      m_lo = (other & 0xFFFFu) > m_lo ? (other & 0xFFFFu) : m_lo;
      m_hi = (other >> 16) > m_hi ? (other >> 16) : m_hi;
      const uint32_t e_lo = mx_biased_exponent(widen_bits<DT>(m_lo)), e_hi = mx_biased_exponent(widen_bits<DT>(m_hi));
      const float sc_lo = bits_f32(e_lo << 23), sc_hi = bits_f32(e_hi << 23);
      uint32_t c[8];
      c[0] = cvt4<DT>(s.a[j][0].x, s.a[j][0].y, sc_lo); c[1] = cvt4<DT>(s.a[j][0].z, s.a[j][0].w, sc_lo);
      c[2] = cvt4<DT>(s.a[j][1].x, s.a[j][1].y, sc_lo); c[3] = cvt4<DT>(s.a[j][1].z, s.a[j][1].w, sc_lo);
      c[4] = cvt4<DT>(s.a[j][2].x, s.a[j][2].y, sc_hi); c[5] = cvt4<DT>(s.a[j][2].z, s.a[j][2].w, sc_hi);
      c[6] = cvt4<DT>(s.a[j][3].x, s.a[j][3].y, sc_hi); c[7] = cvt4<DT>(s.a[j][3].z, s.a[j][3].w, sc_hi);
      if ((a0 | a1 | a2 | a3) >= inf16<DT>()) {  // perhaps an infinity or a NaN among this lane's elements (rare)
#pragma unroll
        for (int h = 0; h < 4; ++h) {
          if ((h == 0 ? a0 : h == 1 ? a1 : h == 2 ? a2 : a3) >= inf16<DT>()) {
            c[2 * h] = nonfinite_fix<DT>(nonfinite_fix<DT>(c[2 * h], s.a[j][h].x, 0), s.a[j][h].y, 16);
            c[2 * h + 1] = nonfinite_fix<DT>(nonfinite_fix<DT>(c[2 * h + 1], s.a[j][h].z, 0), s.a[j][h].w, 16);
          }
        }
      }
      // lane g supplies the exponent of block g: blocks 0, 1 are the low halves of lanes g' = 0-1 and
      // 2-3, blocks 2, 3 their high halves
      const uint32_t got = (uint32_t)__shfl((int)(e_lo | (e_hi << 8)), r16 + 16 * ((g & 1) * 2));
      const int xscale = (int)((g < 2 ? got : got >> 8) & 0xFFu);
      const v8i xf = v8i{(int)c[0], (int)c[1], (int)c[2], (int)c[3], (int)c[4], (int)c[5], (int)c[6], (int)c[7]};
#pragma unroll
      for (int t = 0; t < TN; ++t)  // MFMA rows come from B (output columns n), MFMA columns from x (tokens m)
        acc[t][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[t], xf, acc[t][j], 0, 0, 0, wscale[t], 0, xscale);
    }
  };

  // K steps wave, wave + WAVES, ...: the slabs of the next DEPTH - 1 steps are in flight while this one
  // is multiplied (a ring of register slabs, walked by a loop unrolled over the ring)
  constexpr int DEPTH = TM == 1 ? 4 : 2;
  Slab ring[DEPTH];
#pragma unroll
  for (int d = 0; d + 1 < DEPTH; ++d)
    if (wave + WAVES * d < nk) load(ring[d], wave + WAVES * d);
  int ks = wave;
  while (ks < nk) {
    static_for<DEPTH>([&](auto d_tag) __attribute__((always_inline)) {
      constexpr int d = decltype(d_tag)::value;
      if (ks < nk) {
        const int ahead = ks + WAVES * (DEPTH - 1);
        if (ahead < nk) load(ring[(d + DEPTH - 1) % DEPTH], ahead);
        compute(ring[d]);
        ks += WAVES;
      }
    });
  }

#pragma unroll
  for (int t = 0; t < TN; ++t)
#pragma unroll
    for (int j = 0; j < TM; ++j) partial[wave][t * TM + j][lane] = make_float4(acc[t][j][0], acc[t][j][1], acc[t][j][2], acc[t][j][3]);
  __syncthreads();
  // tile i of the TM * TN is summed and stored by wavefront i % WAVES: lane (r16, g) holds C[m][n .. n+3]
#pragma unroll
  for (int i = 0; i < TM * TN; ++i) {
    if (i % WAVES != wave) continue;
    const int t = i / TM, j = i % TM;
    const int m = m0 + j * 16 + r16, n = n0 + t * 16 + 4 * g;
    if (m >= M) continue;
    float4 v = partial[0][i][lane];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) {
      const float4 o = partial[w][i][lane];
      v.x += o.x; v.y += o.y; v.z += o.z; v.w += o.w;
    }
    if constexpr (ROW) {
      const float4 cs = *reinterpret_cast<const float4*>(wscales + n);
      v.x *= s_row[j] * cs.x; v.y *= s_row[j] * cs.y; v.z *= s_row[j] * cs.z; v.w *= s_row[j] * cs.w;
    }
    if (bias != nullptr) {
      const uint2 braw = *reinterpret_cast<const uint2*>(bias + n);
      v.x += unpack1<OUT>(braw.x & 0xFFFFu); v.y += unpack1<OUT>(braw.x >> 16);
      v.z += unpack1<OUT>(braw.y & 0xFFFFu); v.w += unpack1<OUT>(braw.y >> 16);
    }
    *reinterpret_cast<uint2*>(C + (int64_t)m * N + n) = make_uint2(pack2<OUT>(v.x, v.y), pack2<OUT>(v.z, v.w));
  }
}

template <int DT, int TM, int TN, int MODE>
static void launch_fused(const void* x, int64_t ldx, const void* b, const void* bs, const float* wscales, const void* bias, void* c,
                         int M, int N, int K, hipStream_t st) {
  const dim3 grid((unsigned)(N / (16 * TN)), (unsigned)((M + 16 * TM - 1) / (16 * TM)));
  constexpr int WAVES = TM == 1 ? 8 : 4;
  hipLaunchKernelGGL((gemm_mx_fused_kernel<DT, DT, TM, TN, MODE, WAVES>), grid, dim3(64 * WAVES), 0, st, (const uint16_t*)x, ldx, (const uint8_t*)b,
                     (const uint8_t*)bs, wscales, (const uint16_t*)bias, (uint16_t*)c, M, N, K);
}

// 64-column workgroups when N allows: half as many of them quantize x again, and the weight still
// streams through 144 workgroups at N = 9216 (measured: 32 columns 13.7 us, 64 columns 11.2 us,
// 128 columns 16.7 us at M = 16, K3072 N9216).
template <int DT, int MODE>
static void dispatch_fused(const void* x, int64_t ldx, const void* b, const void* bs, const float* wscales, const void* bias,
                           void* c, int M, int N, int K, hipStream_t st) {
  const int tiles = (M + 15) / 16;
  if (N % 64 == 0) {
    if (tiles <= 1) return launch_fused<DT, 1, 4, MODE>(x, ldx, b, bs, wscales, bias, c, M, N, K, st);
    if (tiles == 2) return launch_fused<DT, 2, 4, MODE>(x, ldx, b, bs, wscales, bias, c, M, N, K, st);
    if (tiles == 3) return launch_fused<DT, 3, 4, MODE>(x, ldx, b, bs, wscales, bias, c, M, N, K, st);
    return launch_fused<DT, 4, 4, MODE>(x, ldx, b, bs, wscales, bias, c, M, N, K, st);
  }
  if (tiles <= 1) return launch_fused<DT, 1, 2, MODE>(x, ldx, b, bs, wscales, bias, c, M, N, K, st);
  if (tiles == 2) return launch_fused<DT, 2, 2, MODE>(x, ldx, b, bs, wscales, bias, c, M, N, K, st);
  if (tiles == 3) return launch_fused<DT, 3, 2, MODE>(x, ldx, b, bs, wscales, bias, c, M, N, K, st);
  return launch_fused<DT, 4, 2, MODE>(x, ldx, b, bs, wscales, bias, c, M, N, K, st);
}

static int check_fused(const char* who, const void* x, int64_t stride_row, const void* b, const void* scales, const void* bias,
                       void* c, int64_t M, int64_t N, int64_t K, int dtype, int scale_align) {
  static thread_local char msg[200];
  auto fail = [&](int code, const char* what) {
    snprintf(msg, sizeof msg, "%s: %s", who, what);
    return km_fail(code, msg);
  };
  if (dtype != KM_BF16 && dtype != KM_F16) return fail(KM_ERR_ARG, "dtype must be bf16 or f16");
  if (M < 0 || N < 0 || K <= 0 || K % kStepBytes) return fail(KM_ERR_UNSUPPORTED, "K must be a positive multiple of 128");
  if (N % kFusedBN) return fail(KM_ERR_UNSUPPORTED, "N must be a multiple of 32");
  if (M * K > 0x7FFFFFFFll || N * K > 0x7FFFFFFFll || (M + 15) / 16 > 65535ll * kFusedMaxTM) return fail(KM_ERR_ARG, "dimension too large");
  if (M == 0 || N == 0) return KM_OK;
  if (!x || !b || !scales || !c) return fail(KM_ERR_ARG, "null pointer");
  if (stride_row < K || stride_row % 8 || ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(b)) & 15) ||
      (reinterpret_cast<uintptr_t>(scales) & (scale_align - 1)) || (reinterpret_cast<uintptr_t>(bias) & 7) || (reinterpret_cast<uintptr_t>(c) & 7))
    return fail(KM_ERR_UNSUPPORTED, "x rows and B must be 16-byte aligned, bias and output 8-byte aligned, scales 8 (mx) / 16 (row) / 4 (block) bytes");
  return KM_OK;
}

}  // namespace km

using namespace km;

extern "C" int km_gemm_mx_fused(const void* x, int64_t stride_row, const void* b, const void* b_scale_packed, const void* bias,
                                void* c, int64_t M, int64_t N, int64_t K, int dtype, void* stream) {
  const int rc = check_fused("km_gemm_mx_fused", x, stride_row, b, b_scale_packed, bias, c, M, N, K, dtype, 8);
  if (rc != KM_OK || M == 0 || N == 0) return rc;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == KM_BF16) dispatch_fused<KM_BF16, kFusedMx>(x, stride_row, b, b_scale_packed, nullptr, bias, c, (int)M, (int)N, (int)K, st);
  else dispatch_fused<KM_F16, kFusedMx>(x, stride_row, b, b_scale_packed, nullptr, bias, c, (int)M, (int)N, (int)K, st);
  return km_check_launch("km_gemm_mx_fused");
}

extern "C" int km_gemm_fp8_rows_fused(const void* x, int64_t stride_row, const void* b, const float* b_scale, const void* bias,
                                      void* c, int64_t M, int64_t N, int64_t K, int dtype, void* stream) {
  const int rc = check_fused("km_gemm_fp8_rows_fused", x, stride_row, b, b_scale, bias, c, M, N, K, dtype, 16);
  if (rc != KM_OK || M == 0 || N == 0) return rc;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == KM_BF16) dispatch_fused<KM_BF16, kFusedRow>(x, stride_row, b, nullptr, b_scale, bias, c, (int)M, (int)N, (int)K, st);
  else dispatch_fused<KM_F16, kFusedRow>(x, stride_row, b, nullptr, b_scale, bias, c, (int)M, (int)N, (int)K, st);
  return km_check_launch("km_gemm_fp8_rows_fused");
}

extern "C" int km_gemm_fp8_blocks_fused(const void* x, int64_t stride_row, const void* b, const float* b_scale, const void* bias,
                                        void* c, int64_t M, int64_t N, int64_t K, int dtype, void* stream) {
  const int rc = check_fused("km_gemm_fp8_blocks_fused", x, stride_row, b, b_scale, bias, c, M, N, K, dtype, 4);
  if (rc != KM_OK || M == 0 || N == 0) return rc;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == KM_BF16) dispatch_fused<KM_BF16, kFusedBlock>(x, stride_row, b, nullptr, b_scale, bias, c, (int)M, (int)N, (int)K, st);
  else dispatch_fused<KM_F16, kFusedBlock>(x, stride_row, b, nullptr, b_scale, bias, c, (int)M, (int)N, (int)K, st);
  return km_check_launch("km_gemm_fp8_blocks_fused");
}
