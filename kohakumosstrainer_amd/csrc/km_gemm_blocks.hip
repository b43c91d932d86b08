// fp8 GEMM of the `block` recipe for gfx950: one fp32 scale per activation row and 128 columns
// of K, one per 128 x 128 block of the weight:
//
//   C[m,n] = sum_kb (A[m, kb] . B[n, kb]) * sa[m, kb] * sb[n / 128, kb]  (+ bias[n])
//
// A [M,K] and B [N,K] e4m3fn with K contiguous, sa [M, K/128] and sb [ceil(N/128), K/128] fp32.
// The partial product of every K block is taken on the fp8 MFMA (fp32 accumulation inside the
// block), multiplied by the two scales and added to the running fp32 sum on the vector ALU: the
// scales are arbitrary fp32 numbers, so they cannot ride on the MFMA's power-of-two scale inputs.
// Replaces the reference's Triton _promote_kernel with SUB = 128, B_ROWS = 128
// (src/kohakumoss_kernels/backends/triton/fp8/gemm.py:108-134,205-216).
//
// Shape of the kernel. A workgroup of four wavefronts (2 x 2) owns a 128 x 128 tile, so the
// weight scale is one number per workgroup and K step; a wavefront's 64 x 64 sub-tile is 16 MFMA
// tiles: 64 registers of partial sums and 64 of running sums per lane, which leaves room for two
// workgroups per compute unit (one's vector-ALU promotion runs under the other's MFMAs). The
// operand slabs of step k+1 are requested (direct-to-LDS buffer loads, double buffered, the
// swizzled slab layout of the other fp8 GEMMs) before the MFMAs of step k are issued and waited
// for after them.
#include <stdio.h>

#include "km_gemm_common.h"

namespace km {

constexpr int kBlkTile = 128;

template <int OUT>
__global__ __launch_bounds__(256, 2) void gemm_fp8_blocks_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, const float* __restrict__ sa,
    const float* __restrict__ sb, const uint16_t* __restrict__ bias, uint16_t* __restrict__ C, int M, int N, int K) {
  constexpr int BM = kBlkTile, BN = kBlkTile;
  constexpr int TM = BM / 32, TN = BN / 32;  // 16x16 MFMA tiles per wavefront and axis
  constexpr int SLAB = BM * kStepBytes;      // 16 KiB
  constexpr int PASSES = BM / 32;            // 4 KiB (32 rows) per pass of 256 lanes
  __shared__ __attribute__((aligned(1024))) uint8_t a_buf0[SLAB];
  __shared__ __attribute__((aligned(1024))) uint8_t a_buf1[SLAB];
  __shared__ __attribute__((aligned(1024))) uint8_t b_buf0[SLAB];
  __shared__ __attribute__((aligned(1024))) uint8_t b_buf1[SLAB];

  int tile_m, tile_n;
  tile_of(blockIdx.x, (M + BM - 1) / BM, (N + BN - 1) / BN, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = (wave >> 1) * (BM / 2), wn = (wave & 1) * (BN / 2);
  const int r16 = lane & 15, g = lane >> 4;
  const int nk = K / kStepBytes;

  // rows past the end are fetched as zeros by the descriptors' range check
  const v4i a_rsrc = raw_rsrc(A + (size_t)m0 * K, (uint32_t)min((int64_t)(M - m0) * K, (int64_t)0x7FFFFFFF));
  const v4i b_rsrc = raw_rsrc(B + (size_t)n0 * K, (uint32_t)min((int64_t)(N - n0) * K, (int64_t)0x7FFFFFFF));
  // staging map of a pass: 8 lanes per row; 16 lanes cover rows r and r+8 (one LDS line)
  const int w = tid >> 3;
  const int srow = ((w >> 4) << 4) + ((w & 1) << 3) + ((w >> 1) & 7);
  const int src_chunk = (tid & 7) ^ (srow & 7);
  const int ld_voff = srow * K + src_chunk * 16;
  const int pass_stride = 32 * K;
  auto dma = [&](uint8_t* abuf, uint8_t* bbuf, int ks) __attribute__((always_inline)) {
    const int koff = __builtin_amdgcn_readfirstlane(ks * kStepBytes);
#pragma unroll
    for (int i = 0; i < PASSES; ++i) hidden_dma_b128(a_rsrc, lds_offset(abuf) + i * 4096 + wave * 1024, ld_voff + i * pass_stride, koff);
#pragma unroll
    for (int i = 0; i < PASSES; ++i) hidden_dma_b128(b_rsrc, lds_offset(bbuf) + i * 4096 + wave * 1024, ld_voff + i * pass_stride, koff);
  };
  auto fragment = [&](const uint8_t* slab, int row) __attribute__((always_inline)) -> v8i {
    const v4i lo = *reinterpret_cast<const v4i*>(slab + slab_offset(row, g));
    const v4i hi = *reinterpret_cast<const v4i*>(slab + slab_offset(row, g + 4));
    return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };

  // scales of this lane's TM token rows (clamped to the last row) and of the tile's weight block
  const float* sa_row[TM];
#pragma unroll
  for (int j = 0; j < TM; ++j) sa_row[j] = sa + (size_t)min(m0 + wm + j * 16 + r16, M - 1) * nk;
  const float* sb_row = sb + (size_t)tile_n * nk;

  v4f acc[TN][TM];
#pragma unroll
  for (int t = 0; t < TN; ++t)
#pragma unroll
    for (int j = 0; j < TM; ++j) acc[t][j] = v4f{0.f, 0.f, 0.f, 0.f};

  // raw scales of the step ahead: loaded a step early, multiplied once that step begins
  float sa_next[TM], sb_next = sb_row[0];
#pragma unroll
  for (int j = 0; j < TM; ++j) sa_next[j] = sa_row[j][0];
  dma(a_buf0, b_buf0, 0);
  __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));
  __syncthreads();

  auto step = [&](const uint8_t* a_cur, const uint8_t* b_cur, uint8_t* a_nxt, uint8_t* b_nxt, int ks) __attribute__((always_inline)) {
    float s_cur[TM];
#pragma unroll
    for (int j = 0; j < TM; ++j) s_cur[j] = sa_next[j] * sb_next;
    if (ks + 1 < nk) {
      // the other pair of buffers was last read in the step before, behind that step's barrier
      sb_next = sb_row[ks + 1];
#pragma unroll
      for (int j = 0; j < TM; ++j) sa_next[j] = sa_row[j][ks + 1];
      dma(a_nxt, b_nxt, ks + 1);
    }
    v8i xf[TM];
#pragma unroll
    for (int j = 0; j < TM; ++j) xf[j] = fragment(a_cur, wm + j * 16 + r16);
    v8i wf = fragment(b_cur, wn + r16);
    // The four MFMAs of a row of tiles are issued back to back; the sums of the row before are
    // promoted on the vector ALU while they run (two sets of partial-sum registers).
    v4f part[2][TM];
    static_for<TN + 1>([&](auto t_tag) __attribute__((always_inline)) {
      constexpr int t = decltype(t_tag)::value;
      if constexpr (t < TN) {
        v8i wf_next = wf;
        if constexpr (t + 1 < TN) wf_next = fragment(b_cur, wn + (t + 1) * 16 + r16);
#pragma unroll
        for (int j = 0; j < TM; ++j) {
          // MFMA rows come from B (output columns n), MFMA columns from A (tokens m); unit scales
          part[t & 1][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, xf[j], v4f{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
        }
        wf = wf_next;
      }
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (t > 0) {
#pragma unroll
        for (int j = 0; j < TM; ++j) {
#pragma unroll
          for (int v = 0; v < 4; ++v) acc[t - 1][j][v] = __builtin_fmaf(part[(t - 1) & 1][j][v], s_cur[j], acc[t - 1][j][v]);
          // pins the promotion ahead of the wait below (the compiler would sink it past the barrier)
          asm volatile("" : "+v"(acc[t - 1][j]));
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));  // the slabs of the next step have landed, this step's LDS reads are done
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
  };
  for (int ks = 0; ks < nk; ks += 2) {
    step(a_buf0, b_buf0, a_buf1, b_buf1, ks);
    if (ks + 1 < nk) step(a_buf1, b_buf1, a_buf0, b_buf0, ks + 1);
  }

  store_tile<BM, BN, OUT, 0>(acc, 1.0f, nullptr, nullptr, bias, C, M, N, m0, n0, a_buf0, a_buf1, b_buf0, b_buf1);
}

int blocks_gemm_num_configs() { return 1; }
int blocks_gemm_config_desc(int config, char* buf, int len) {
  if (config != 0) return km_fail(KM_ERR_ARG, "config out of range");
  snprintf(buf, len, "bm=%d,bn=%d,bk=128,waves=4,wg_per_cu=2", kBlkTile, kBlkTile);
  return KM_OK;
}

}  // namespace km

using namespace km;

extern "C" int km_gemm_fp8_blocks(const void* a, const float* sa, const void* b, const float* sb,
                                  const void* bias, void* c, int64_t M, int64_t N, int64_t K,
                                  int out_dtype, int config, void* stream) {
  if (out_dtype != KM_BF16 && out_dtype != KM_F16) return km_fail(KM_ERR_ARG, "km_gemm_fp8_blocks: out_dtype must be bf16 or f16");
  if (M < 0 || N < 0 || K <= 0 || K % kStepBytes) return km_fail(KM_ERR_UNSUPPORTED, "km_gemm_fp8_blocks: K must be a positive multiple of 128");
  if (M * K > 0x7FFFFFFFll || N * K > 0x7FFFFFFFll || M > 0x0FFFFFFF || N > 0x0FFFFFFF)
    return km_fail(KM_ERR_ARG, "km_gemm_fp8_blocks: dimension too large");
  if (config != 0) return km_fail(KM_ERR_ARG, "km_gemm_fp8_blocks: config out of range");
  if (M == 0 || N == 0) return KM_OK;
  if (!a || !b || !c || !sa || !sb) return km_fail(KM_ERR_ARG, "km_gemm_fp8_blocks: null pointer");
  if ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15)
    return km_fail(KM_ERR_UNSUPPORTED, "km_gemm_fp8_blocks: operands must be 16-byte aligned");
  const int tiles = (int)(((M + kBlkTile - 1) / kBlkTile) * ((N + kBlkTile - 1) / kBlkTile));
  hipStream_t st = (hipStream_t)stream;
  if (out_dtype == KM_BF16)
    hipLaunchKernelGGL(gemm_fp8_blocks_kernel<KM_BF16>, dim3(tiles), dim3(256), 0, st, (const uint8_t*)a, (const uint8_t*)b, sa, sb,
                       (const uint16_t*)bias, (uint16_t*)c, (int)M, (int)N, (int)K);
  else
    hipLaunchKernelGGL(gemm_fp8_blocks_kernel<KM_F16>, dim3(tiles), dim3(256), 0, st, (const uint8_t*)a, (const uint8_t*)b, sa, sb,
                       (const uint16_t*)bias, (uint16_t*)c, (int)M, (int)N, (int)K);
  return km_check_launch("km_gemm_fp8_blocks");
}
