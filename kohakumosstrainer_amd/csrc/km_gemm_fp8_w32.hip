// The fp8 GEMMs of km_gemm_fp8.hip on the larger block-scaled MFMA, V_MFMA_SCALE_F32_32X32X64_F8F6F4:
//
//   C[M,N] = A[M,K] B[N,K]^T (+ bias), A and B e4m3fn with K contiguous, fp32 accumulation over all
//   of K, scales applied by the MFMA (mx) or on the accumulator (tensor, row), one rounding.
//
// Same slabs, same direct-to-LDS fetch schedule and the same roles as gemm_fp8_kernel (reference
// kernels: src/kohakumoss_kernels/backends/triton/fp8/gemm.py:66-171): a workgroup of four
// wavefronts owns a 256 x 256 tile, walks K in steps of 128 bytes, keeps the A fragments of a
// step in registers and streams the B fragments. What changes is the instruction: a 32 x 32 tile
// over 64 K bytes does twice the work of the 16 x 16 x 128 one and occupies the matrix pipe for
// 64 cycles instead of 32, so a wavefront issues half as many of them per step and every
// instruction it threads between two MFMAs (a direct-to-LDS fetch with its m0 write, a pair of
// fragment reads, a wait) has twice the time to issue before the pipe runs dry. On one compute
// unit the four wavefronts share one path to memory; a fetch that waits its turn there for more
// than 32 cycles stalls the 16 x 16 pipeline and not this one.
//
// Operand layout of the 32x32x64 MFMA (measured with random operands against the exact product):
// lane l carries, for row l%32 and h = l/32, the K bytes [16h, 16h+16) in its first four registers
// and [32+16h, 32+16h+16) in its last four; the E8M0 byte of lane l scales K block h (bytes
// [32h, 32h+32)) of row l%32. Output: lane l holds D[8*(v/4) + 4*(l/32) + v%4][l%32], v = 0..15.
// A K step of 128 bytes is two such instructions per tile (K halves c = 0, 1); a slab row's chunks
// 4c+h and 4c+2+h are the lane's two register halves, its scale is block 2c+h of the step.
#include <stdio.h>

#include "km_gemm_common.h"

namespace km {

typedef float v16f __attribute__((ext_vector_type(16)));

// c += A(32x64) * B(64x32), block scaled, accumulating in place in 16 AGPRs. BYTE_A / BYTE_B (0 or
// 2) pick the byte of each scale register: op_sel is the low bit of the byte index, op_sel_hi the high.
#define KM_MFMA32_ASM(OHA, OHB)                                                                                      \
  asm("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:[0,0,0] op_sel_hi:[" #OHA "," #OHB ",0]"     \
      : "+a"(c)                                                                                                      \
      : "v"(a), "v"(b), "v"(sa), "v"(sb))
template <int BYTE_A, int BYTE_B>
__device__ __forceinline__ void mfma32_acc(v16f& c, const v8i& a, const v8i& b, int sa, int sb) {
  static_assert((BYTE_A == 0 || BYTE_A == 2) && (BYTE_B == 0 || BYTE_B == 2), "scale bytes 0 and 2");
  if constexpr (BYTE_A == 0 && BYTE_B == 0) KM_MFMA32_ASM(0, 0);
  else if constexpr (BYTE_A == 0) KM_MFMA32_ASM(0, 1);
  else if constexpr (BYTE_B == 0) KM_MFMA32_ASM(1, 0);
  else KM_MFMA32_ASM(1, 1);
}
#undef KM_MFMA32_ASM

// Epilogue for accumulators in the 32 x 32 layout: acc[t][j][v] of lane (r = lane%32, h = lane/32)
// is C[m0 + wm + 32j + r][n0 + wn + 32t + 8*(v/4) + 4h + v%4]. Same arithmetic and the same
// LDS transpose to full-line stores as store_tile. SCALED 0: acc + bias; 1: acc * (post * row
// scale * column scale) + bias.
template <int OUT, int SCALED>
__device__ __forceinline__ void store_tile32(v16f (&acc)[4][4], float post, const float* __restrict__ row_scale,
                                             const float* __restrict__ col_scale, const uint16_t* __restrict__ bias,
                                             uint16_t* __restrict__ C, int M, int N, int m0, int n0, uint8_t* buf0,
                                             uint8_t* buf1, uint8_t* buf2, uint8_t* buf3) {
  constexpr int BM = 256, BN = 256, WT = 128;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) & 3;
  const int wm = (wave >> 1) * WT, wn = (wave & 1) * WT;
  const int r = lane & 31, h = lane >> 5;
  const bool has_bias = bias != nullptr;
  auto value = [&](float a, float s, float b) __attribute__((always_inline)) {
    if constexpr (SCALED == 1) return a * s + b;
    else return a + b;
  };
  if (m0 + BM <= M && n0 + BN <= N && (N & 7) == 0) {
    constexpr int RP = WT * 2 + 16;  // LDS row pitch in bytes
    constexpr int HM = 2;            // 32-row tiles per pass: 64 rows x 272 B fit one 32 KiB buffer
    constexpr int LPR = WT * 2 / 16, RPI = 64 / LPR;
    __syncthreads();  // every wavefront is done reading fragments
    uint8_t* region = wave == 0 ? buf0 : wave == 1 ? buf1 : wave == 2 ? buf2 : buf3;
    // bias and column scales of the lane's 16 groups of 4 columns: group (t, q) starts at 32t + 8q + 4h
    uint2 braw[4][4];
    float4 cs[SCALED == 1 ? 4 : 1][SCALED == 1 ? 4 : 1];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + wn + 32 * t + 8 * q + 4 * h;
        braw[t][q] = has_bias ? *reinterpret_cast<const uint2*>(bias + n) : make_uint2(0u, 0u);
        if constexpr (SCALED == 1) cs[t][q] = col_scale != nullptr ? *reinterpret_cast<const float4*>(col_scale + n) : make_float4(1.f, 1.f, 1.f, 1.f);
      }
    uint8_t* out_base = reinterpret_cast<uint8_t*>(C) + ((size_t)(m0 + wm) * N + n0 + wn) * 2;
    const int rd_row = lane / LPR, rd_col = (lane % LPR) * 16;
    static_for<4 / HM>([&](auto p_tag) __attribute__((always_inline)) {
      constexpr int pass = decltype(p_tag)::value;
      static_for<HM>([&](auto j_tag) __attribute__((always_inline)) {
        constexpr int jj = decltype(j_tag)::value;
        constexpr int j = pass * HM + jj;
        const float rs = (SCALED == 1 && row_scale != nullptr) ? post * row_scale[m0 + wm + 32 * j + r] : post;
        static_for<4>([&](auto t_tag) __attribute__((always_inline)) {
          constexpr int t = decltype(t_tag)::value;
          static_for<4>([&](auto q_tag) __attribute__((always_inline)) {
            constexpr int q = decltype(q_tag)::value;
            const float b0 = unpack1<OUT>(braw[t][q].x & 0xFFFFu), b1 = unpack1<OUT>(braw[t][q].x >> 16);
            const float b2 = unpack1<OUT>(braw[t][q].y & 0xFFFFu), b3 = unpack1<OUT>(braw[t][q].y >> 16);
            float s0 = rs, s1 = rs, s2 = rs, s3 = rs;
            if constexpr (SCALED == 1) {
              s0 = rs * cs[t][q].x; s1 = rs * cs[t][q].y; s2 = rs * cs[t][q].z; s3 = rs * cs[t][q].w;
            }
            const float o0 = value(acc[t][j][4 * q + 0], s0, b0), o1 = value(acc[t][j][4 * q + 1], s1, b1);
            const float o2 = value(acc[t][j][4 * q + 2], s2, b2), o3 = value(acc[t][j][4 * q + 3], s3, b3);
            *reinterpret_cast<uint2*>(region + (jj * 32 + r) * RP + (32 * t + 8 * q + 4 * h) * 2) =
                make_uint2(pack2<OUT>(o0, o1), pack2<OUT>(o2, o3));
          });
        });
      });
      // only this wavefront touches its region: LDS operations of one wavefront stay in order
      static_for<HM * 32 / RPI>([&](auto i_tag) __attribute__((always_inline)) {
        constexpr int i = decltype(i_tag)::value;
        const int row = i * RPI + rd_row;
        const uint4 v = *reinterpret_cast<const uint4*>(region + row * RP + rd_col);
        __builtin_nontemporal_store(__builtin_bit_cast(v4i, v), reinterpret_cast<v4i*>(out_base + (size_t)(pass * HM * 32 + row) * N * 2 + rd_col));
      });
    });
    return;
  }
  const bool vec_ok = (N & 3) == 0;
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int n = n0 + wn + 32 * t + 8 * q + 4 * h;
      float bv[4] = {0.f, 0.f, 0.f, 0.f}, cv[4] = {1.f, 1.f, 1.f, 1.f};
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        if (has_bias && n + v < N) bv[v] = unpack1<OUT>(bias[n + v]);
        if (SCALED == 1 && col_scale != nullptr && n + v < N) cv[v] = col_scale[n + v];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int m = m0 + wm + 32 * j + r;
        if (m >= M || n >= N) continue;
        const float rs = (SCALED == 1 && row_scale != nullptr) ? post * row_scale[m] : post;
        float o[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) o[v] = value(acc[t][j][4 * q + v], rs * cv[v], bv[v]);
        uint16_t* dst = C + (size_t)m * N + n;
        if (vec_ok && n + 3 < N) {
          *reinterpret_cast<uint2*>(dst) = make_uint2(pack2<OUT>(o[0], o[1]), pack2<OUT>(o[2], o[3]));
        } else {
#pragma unroll
          for (int v = 0; v < 4; ++v)
            if (n + v < N) dst[v] = (uint16_t)(pack2<OUT>(o[v], 0.f) & 0xFFFFu);
        }
      }
    }
}

template <bool MX, bool SCALE_KM, int OUT>
__global__ __launch_bounds__(256, 1) void gemm_fp8_w32_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ As, const uint8_t* __restrict__ B,
    const uint8_t* __restrict__ Bs, const float* __restrict__ sa, const float* __restrict__ sb,
    const uint16_t* __restrict__ bias, uint16_t* __restrict__ C, int M, int N, int K, int scale_vectors) {
  constexpr int BM = 256, BN = 256, WT = 128;
  constexpr int SLAB = BM * kStepBytes;  // 32 KiB per operand and stage
  constexpr int LD = BM / 32;            // direct-to-LDS passes of 32 rows per slab
  constexpr int kWaitAllButA = wait_vm_lgkm0(LD);
  __shared__ __attribute__((aligned(1024))) uint8_t a_buf0[SLAB];
  __shared__ __attribute__((aligned(1024))) uint8_t a_buf1[SLAB];
  __shared__ __attribute__((aligned(1024))) uint8_t b_buf0[SLAB];
  __shared__ __attribute__((aligned(1024))) uint8_t b_buf1[SLAB];

  int tile_m, tile_n;
  tile_of(blockIdx.x, (M + BM - 1) / BM, (N + BN - 1) / BN, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = (wave >> 1) * WT, wn = (wave & 1) * WT;
  const int r32 = lane & 31, h = lane >> 5;
  const int nk = K / kStepBytes;
  const int kb = K >> 5;  // scale bytes per row (natural layout)

  const v4i a_rsrc = raw_rsrc(A + (size_t)m0 * K, (uint32_t)min((int64_t)(M - m0) * K, (int64_t)0x7FFFFFFF));
  const v4i b_rsrc = raw_rsrc(B + (size_t)n0 * K, (uint32_t)min((int64_t)(N - n0) * K, (int64_t)0x7FFFFFFF));
  // staging map of a pass: 8 lanes per row; 16 lanes cover rows r and r+8 (one LDS line)
  const int w = tid >> 3;
  const int srow = ((w >> 4) << 4) + ((w & 1) << 3) + ((w >> 1) & 7);  // 0 .. 31
  const int src_chunk = (tid & 7) ^ (srow & 7);
  const int ld_voff = srow * K + src_chunk * 16;
  const int pass_stride = 32 * K;

  // Scales. Packed copy (km_scales_pack): for a K step and a group of 128 rows, byte
  // (row%16)*32 + 8*block + (row%128)/16. A lane (row r32 of every 32-row tile, blocks h and 2+h)
  // fetches the 8-byte runs of its two blocks and shifts them by a byte when r32 >= 16: the scale
  // of tile T is then byte 2T of the run. A wavefront's 128 rows are exactly one group.
  v4i ws_rsrc, xs_rsrc;
  int ws_off[SCALE_KM ? 2 : 4], xs_off[SCALE_KM ? 2 : 4];
  int ws_step = 0, xs_step = 0, ws_base = 0, xs_base = 0;
  const int run_shift = (r32 >> 4) * 8;
  if constexpr (MX) {
    if constexpr (SCALE_KM) {
      const int rbn = (N + 127) >> 7, rbm = (M + 127) >> 7;
      ws_rsrc = raw_rsrc(Bs, (uint32_t)min((int64_t)nk * rbn * 512, (int64_t)0x7FFFFFFF));
      xs_rsrc = raw_rsrc(As, (uint32_t)min((int64_t)nk * rbm * 512, (int64_t)0x7FFFFFFF));
      ws_off[0] = xs_off[0] = (r32 & 15) * 32 + h * 8;
      ws_off[1] = xs_off[1] = ws_off[0] + 16;
      ws_base = min((n0 + wn) >> 7, rbn - 1) * 512;  // wavefronts wholly past the edge read valid bytes
      xs_base = min((m0 + wm) >> 7, rbm - 1) * 512;
      ws_step = rbn * 512;
      xs_step = rbm * 512;
    } else {
      ws_rsrc = raw_rsrc(Bs + (size_t)n0 * kb, (uint32_t)min((int64_t)(N - n0) * kb, (int64_t)0x7FFFFFFF));
      xs_rsrc = raw_rsrc(As + (size_t)m0 * kb, (uint32_t)min((int64_t)(M - m0) * kb, (int64_t)0x7FFFFFFF));
      ws_step = xs_step = 4;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        ws_off[t] = min(wn + t * 32 + r32, N - 1 - n0) * kb;
        xs_off[t] = min(wm + t * 32 + r32, M - 1 - m0) * kb;
      }
    }
  }

  v16f acc[4][4];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[t][j][v] = 0.f;

  v8i xf[4][2];  // A fragments of the step: tile j, K half c
  v8i wcur;
  // Scale operands per step parity, K half and (packed) pair of tiles / (natural) tile; a step
  // reads its own set while the next step's is written (the MFMAs are opaque to the compiler's
  // hazard handling, so a register an MFMA may still read is never rewritten).
  constexpr int NS = SCALE_KM ? 2 : 4;
  int wsc[2][2][NS], xsc[2][2][NS];
  uint64_t wraw64[2] = {0, 0}, xraw64[2] = {0, 0};
  uint32_t wraw32[4], xraw32[4];

  auto dma_a_pass = [&](uint32_t buf, int koff, int i) __attribute__((always_inline)) {
    hidden_dma_b128(a_rsrc, buf + i * 4096 + wave * 1024, ld_voff + i * pass_stride, koff);
  };
  auto dma_b_pass = [&](uint32_t buf, int koff, int i) __attribute__((always_inline)) {
    hidden_dma_b128(b_rsrc, buf + i * 4096 + wave * 1024, ld_voff + i * pass_stride, koff);
  };
  auto scale_fetch = [&](int ks) __attribute__((always_inline)) {
    if constexpr (MX) {
      const int wso = __builtin_amdgcn_readfirstlane(ks * ws_step + ws_base);
      const int xso = __builtin_amdgcn_readfirstlane(ks * xs_step + xs_base);
      if constexpr (SCALE_KM) {
#pragma unroll
        for (int c = 0; c < 2; ++c) {
          wraw64[c] = hidden_load_b64(ws_rsrc, ws_off[c], wso);
          xraw64[c] = hidden_load_b64(xs_rsrc, xs_off[c], xso);
        }
      } else {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          wraw32[t] = hidden_load_b32(ws_rsrc, ws_off[t], wso);
          xraw32[t] = hidden_load_b32(xs_rsrc, xs_off[t], xso);
        }
      }
    }
  };
  constexpr int kScaleLoads = MX ? (SCALE_KM ? 4 : 8) : 0;
  // `live` is all ones for a real step and zero for the padding step of an odd step count: zero
  // scale bytes (2^-127 on both sides) make that step add exactly 0.
  auto scale_commit = [&](auto set_tag, uint32_t live) __attribute__((always_inline)) {
    constexpr int P = decltype(set_tag)::value;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      if constexpr (!MX) {
#pragma unroll
        for (int i = 0; i < NS; ++i) wsc[P][c][i] = xsc[P][c][i] = (int)(0x7F7F7F7Fu & live);
      } else if constexpr (SCALE_KM) {
        const uint64_t wv = wraw64[c] >> run_shift, xv = xraw64[c] >> run_shift;
        wsc[P][c][0] = (int)((uint32_t)wv & live); wsc[P][c][1] = (int)((uint32_t)(wv >> 32) & live);
        xsc[P][c][0] = (int)((uint32_t)xv & live); xsc[P][c][1] = (int)((uint32_t)(xv >> 32) & live);
      } else {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          wsc[P][c][t] = (int)((wraw32[t] >> (8 * h + 16 * c)) & live);
          xsc[P][c][t] = (int)((xraw32[t] >> (8 * h + 16 * c)) & live);
        }
      }
    }
  };
  typedef __attribute__((address_space(3))) const v4i* lds_v4i_cptr;
  // fragment of the 32 rows from `row0` on, K half c: chunks 4c+h and 4c+2+h of row row0 + r32
  auto fragment = [&](uint32_t slab, int row0, int c) __attribute__((always_inline)) -> v8i {
    const v4i lo = *(lds_v4i_cptr)(slab + slab_offset(row0 + r32, 4 * c + h));
    const v4i hi = *(lds_v4i_cptr)(slab + slab_offset(row0 + r32, 4 * c + 2 + h));
    return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };

  // One K step with scale set P: 8 groups (B tile t, K half c) of 4 MFMAs. A(k) is in registers,
  // B(k) in b_cur. B(k+1) goes to b_nxt and A(k+2) to a_cur between the MFMAs of the first seven
  // groups; before the last group the wavefront waits for B(k+1) (and A(k+1), older), passes the
  // barrier and reads the first fragments of step k+1 behind the last four MFMAs. Each fragment
  // register is reloaded at least one MFMA after the last MFMA that read it.
  constexpr int kWindow = 28;                   // MFMAs before the last group
  constexpr int kBWindow = 10;                  // B passes over the first third, A passes over the rest
  auto step = [&](uint32_t a_cur, uint32_t a_nxt, uint32_t b_cur, uint32_t b_nxt, int ks, auto set_tag) __attribute__((always_inline)) {
    constexpr int P = decltype(set_tag)::value;
    const int next = min(ks + 1, nk - 1);
    const int koff_b = __builtin_amdgcn_readfirstlane(next * kStepBytes);
    const int koff_a = __builtin_amdgcn_readfirstlane(min(ks + 2, nk - 1) * kStepBytes);
    scale_fetch(next);
    __builtin_amdgcn_sched_barrier(0);
    static_for<8>([&](auto g_tag) __attribute__((always_inline)) {
      constexpr int grp = decltype(g_tag)::value;
      constexpr int t = grp >> 1, c = grp & 1;
      v8i wnext;
      if constexpr (grp < 7) {
        wnext = fragment(b_cur, wn + ((grp + 1) >> 1) * 32, (grp + 1) & 1);
      } else {
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(kWaitAllButA);  // B(k+1), scales(k+1) and A(k+1) landed
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        wnext = fragment(b_nxt, wn, 0);
      }
      static_for<4>([&](auto j_tag) __attribute__((always_inline)) {
        constexpr int j = decltype(j_tag)::value;
        constexpr int q = grp * 4 + j;  // position in the step's MFMA sequence
        if constexpr (SCALE_KM || !MX)
          mfma32_acc<(t & 1) * 2 * (MX ? 1 : 0), (j & 1) * 2 * (MX ? 1 : 0)>(acc[t][j], wcur, xf[j][c], wsc[P][c][MX ? t >> 1 : 0], xsc[P][c][MX ? j >> 1 : 0]);
        else
          mfma32_acc<0, 0>(acc[t][j], wcur, xf[j][c], wsc[P][c][t], xsc[P][c][j]);
        if constexpr (grp < 7) {
          static_for<LD>([&](auto i_tag) __attribute__((always_inline)) {
            constexpr int i = decltype(i_tag)::value;
            if constexpr (q == i * kBWindow / LD) {
              __builtin_amdgcn_sched_barrier(0);
              dma_b_pass(b_nxt, koff_b, i);
              __builtin_amdgcn_sched_barrier(0);
            }
          });
          static_for<LD>([&](auto i_tag) __attribute__((always_inline)) {
            constexpr int i = decltype(i_tag)::value;
            if constexpr (q == kBWindow + i * (kWindow - kBWindow) / LD) {
              __builtin_amdgcn_sched_barrier(0);
              if constexpr (i == 0) {
                // a_cur still holds A(k): every wavefront must have read its fragments (at the end
                // of the step before) before the slab is overwritten
                __builtin_amdgcn_s_waitcnt(kWaitLgkm0);
                __syncthreads();
              }
              dma_a_pass(a_cur, koff_a, i);
              __builtin_amdgcn_sched_barrier(0);
            }
          });
        } else {
          // the last group: the K half 0 fragments were last read a group ago, the K half 1
          // fragment of tile j-1 by the MFMA before this one
          __builtin_amdgcn_sched_barrier(0);
          xf[j][0] = fragment(a_nxt, wm + j * 32, 0);
          if constexpr (j >= 1) xf[j - 1][1] = fragment(a_nxt, wm + (j - 1) * 32, 1);
        }
      });
      if constexpr (grp == 7) {
        __builtin_amdgcn_sched_barrier(0);
        xf[3][1] = fragment(a_nxt, wm + 3 * 32, 1);
      }
      wcur = wnext;
    });
    scale_commit(std::integral_constant<int, P ^ 1>{}, ks + 1 < nk ? 0xFFFFFFFFu : 0u);
    __builtin_amdgcn_sched_barrier(0);
  };
  using set0_t = std::integral_constant<int, 0>;
  using set1_t = std::integral_constant<int, 1>;
  static_assert(kScaleLoads + LD <= 63, "vmcnt");

  // prologue: A(0), B(0), A(1) and the scales of step 0
  const uint32_t la0 = lds_offset(a_buf0), la1 = lds_offset(a_buf1), lb0 = lds_offset(b_buf0), lb1 = lds_offset(b_buf1);
  {
    const int k1 = __builtin_amdgcn_readfirstlane(min(1, nk - 1) * kStepBytes);
#pragma unroll
    for (int i = 0; i < LD; ++i) dma_a_pass(la0, 0, i);
#pragma unroll
    for (int i = 0; i < LD; ++i) dma_b_pass(lb0, 0, i);
    scale_fetch(0);
#pragma unroll
    for (int i = 0; i < LD; ++i) dma_a_pass(la1, k1, i);
  }
  __builtin_amdgcn_s_waitcnt(kWaitVm0);
  __syncthreads();
  scale_commit(set0_t{}, 0xFFFFFFFFu);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    xf[j][0] = fragment(la0, wm + j * 32, 0);
    xf[j][1] = fragment(la0, wm + j * 32, 1);
  }
  wcur = fragment(lb0, wn, 0);

  // two steps per trip, one per buffer parity; an odd step count is padded with a zero-scaled step
  const int nsteps = (nk + 1) & ~1;
  for (int ks = 0; ks < nsteps; ks += 2) {
    step(la0, la1, lb0, lb1, ks, set0_t{});
    step(la1, la0, lb1, lb0, ks + 1, set1_t{});
  }
  __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));  // the last (clamped) prefetches and fragment reads are done before LDS is reused

  // the MFMAs above are opaque to the compiler's hazard handling: give the last ones (16 passes
  // each) time to retire before the accumulators are read
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  // The compiler does not know that the opaque MFMAs' results take time and copies accumulators to
  // vector registers wherever it likes (the loop exit included): passing every accumulator through an
  // empty statement placed after the wait makes each later read depend on it.
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) asm volatile("" : "+a"(acc[i][j]));
  __builtin_amdgcn_sched_barrier(0);

  float post = 1.0f;
  const float *row_scale = nullptr, *col_scale = nullptr;
  if constexpr (!MX) {
    if (scale_vectors) {
      row_scale = sa;
      col_scale = sb;
    } else {
      post = sa[0] * sb[0];
    }
  }
  store_tile32<OUT, MX ? 0 : 1>(acc, post, row_scale, col_scale, bias, C, M, N, m0, n0, a_buf0, a_buf1, b_buf0, b_buf1);
}

template <bool MX, bool SCALE_KM, int OUT>
static int launch_w32(const void* a, const void* as, const void* b, const void* bs, const float* sa, const float* sb,
                      const void* bias, void* c, int M, int N, int K, int scale_vectors, hipStream_t st) {
  const int tiles = ((M + 255) / 256) * ((N + 255) / 256);
  hipLaunchKernelGGL((gemm_fp8_w32_kernel<MX, SCALE_KM, OUT>), dim3(tiles), dim3(256), 0, st, (const uint8_t*)a,
                     (const uint8_t*)as, (const uint8_t*)b, (const uint8_t*)bs, sa, sb, (const uint16_t*)bias,
                     (uint16_t*)c, M, N, K, scale_vectors);
  return km_check_launch("km_gemm");
}

// mx: scale_layout packed / natural; tensor and row recipes: mx = false
int gemm_w32(bool mx, bool packed, int out_dtype, const void* a, const void* as, const void* b, const void* bs,
             const float* sa, const float* sb, const void* bias, void* c, int M, int N, int K, int scale_vectors,
             hipStream_t st) {
  const bool bf = out_dtype == KM_BF16;
  if (!mx)
    return bf ? launch_w32<false, false, KM_BF16>(a, as, b, bs, sa, sb, bias, c, M, N, K, scale_vectors, st)
              : launch_w32<false, false, KM_F16>(a, as, b, bs, sa, sb, bias, c, M, N, K, scale_vectors, st);
  if (packed)
    return bf ? launch_w32<true, true, KM_BF16>(a, as, b, bs, sa, sb, bias, c, M, N, K, scale_vectors, st)
              : launch_w32<true, true, KM_F16>(a, as, b, bs, sa, sb, bias, c, M, N, K, scale_vectors, st);
  return bf ? launch_w32<true, false, KM_BF16>(a, as, b, bs, sa, sb, bias, c, M, N, K, scale_vectors, st)
            : launch_w32<true, false, KM_F16>(a, as, b, bs, sa, sb, bias, c, M, N, K, scale_vectors, st);
}

}  // namespace km
