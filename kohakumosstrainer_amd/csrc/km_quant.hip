// Activation / weight quantizers for gfx950: bandwidth kernels.
//
//   quant_mx_rows     MXFP8 along a unit-stride contraction axis (reference
//                     src/kohakumoss_kernels/fp8/formats.py:94-99; the Triton kernel it
//                     replaces is backends/triton/fp8/quantize.py:94-118)
//   quant_cols<MX>    MXFP8 of the transposed view (blocks run along the strided axis of
//                     the input), what `quantize(x.t(), "mx")` computes for the input-
//                     gradient weight copy (reference src/kohakumoss/quant/compute.py:63-66)
//   quant_mx_generic  any strides, one thread per block of 32
//   tensor_amax / tensor_cast   per-tensor recipe (reference formats.py:77-79,
//                     Triton quantize.py:86-91,161-168)
//   quant_i8_rows     int8 per-row quantizer of the int8 compute linear (reference
//                     src/kohakumoss_kernels/int8/formats.py:21-38)
//   quant_fp8_rows    per-row recipe, one fp32 scale per row (reference formats.py:80-82,
//                     Triton quantize.py:64-84,151-158)
//
// All of them read each input element once and write each output byte once.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "km_hadamard_common.h"
#include "km_internal.h"
#include "km_numeric.h"
#include "km_quant_common.h"

namespace km {

// Byte offset of scale (row, block) in the MFMA-packed layout the GEMM reads: per K step of
// 128 and group of 128 rows, 512 bytes ordered [row%16][block%4][row%128/16].
__device__ __forceinline__ uint64_t scale_pack_offset(uint64_t row, uint64_t block, uint64_t row_groups) {
  return ((((block >> 2) * row_groups + (row >> 7)) * 16 + (row & 15)) * 4 + (block & 3)) * 8 + ((row & 127) >> 4);
}

// max over the 4 lanes of a quad, every lane of the quad gets it (DPP quad_perm swaps).
__device__ __forceinline__ uint32_t quad_max(uint32_t v) {
  uint32_t o = (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0xB1, 0xF, 0xF, true);  // [1,0,3,2]
  v = v > o ? v : o;
  o = (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x4E, 0xF, 0xF, true);  // [2,3,0,1]
  return v > o ? v : o;
}

// ---- rows: lane = 8 consecutive elements, quad = one block of 32 --------------------------
// Group g (8 elements) of row g / groups_per_row; outputs are flat because q and the
// scales are contiguous row-major. UNROLL independent 128-bit loads are in flight per lane.
constexpr int kRowsThreads = 256;
constexpr int kRowsUnroll = 4;

// byte of lane i+4, i+8, i+12 of the same 16-lane row gathered into one dword (lane i%16 == 0
// ends up with the four scale bytes of four consecutive blocks)
__device__ __forceinline__ uint32_t gather4_stride4(uint32_t b) {
  uint32_t v = b & 0xFFu;
  v |= ((uint32_t)__builtin_amdgcn_mov_dpp((int)b, 0x104, 0xF, 0xF, true) & 0xFFu) << 8;   // row_shl:4
  v |= ((uint32_t)__builtin_amdgcn_mov_dpp((int)b, 0x108, 0xF, 0xF, true) & 0xFFu) << 16;  // row_shl:8
  v |= ((uint32_t)__builtin_amdgcn_mov_dpp((int)b, 0x10C, 0xF, 0xF, true) & 0xFFu) << 24;  // row_shl:12
  return v;
}

// PACK4: cols % 128 == 0, so the 16 lanes of a DPP row cover four consecutive blocks of one
// row and their natural-layout scale bytes are stored as one dword.
template <int DT, bool PACK4>
__global__ __launch_bounds__(kRowsThreads) void quant_mx_rows(
    const uint16_t* __restrict__ x, int64_t ld, uint32_t groups_per_row, uint64_t ngroups, uint32_t rows,
    uint8_t* __restrict__ q, uint8_t* __restrict__ scales, uint8_t* __restrict__ scales_km) {
  saturating_conversions();
  const uint64_t base = (uint64_t)blockIdx.x * (kRowsThreads * kRowsUnroll) + threadIdx.x;
  const bool dense = ld == (int64_t)groups_per_row * 8;
  uint4 raw[kRowsUnroll];
#pragma unroll
  for (int u = 0; u < kRowsUnroll; ++u) {
    const uint64_t g = base + (uint64_t)u * kRowsThreads;
    raw[u] = make_uint4(0, 0, 0, 0);
    if (g < ngroups) {
      uint64_t off;
      if (dense) {
        off = g * 8;
      } else {
        const uint64_t row = g / groups_per_row;
        off = row * (uint64_t)ld + (g - row * groups_per_row) * 8;
      }
      raw[u] = *reinterpret_cast<const uint4*>(x + off);
    }
  }
#pragma unroll
  for (int u = 0; u < kRowsUnroll; ++u) {
    const uint64_t g = base + (uint64_t)u * kRowsThreads;
    const uint32_t m16 = amax16x8(raw[u]);
    const uint32_t biased = mx_biased_exponent(quad_max(widen_bits<DT>(m16)));
    const float sc = bits_f32(biased << 23);  // 2^(biased - 127) as the conversion's scale operand
    uint2 codes = make_uint2(cvt4<DT>(raw[u].x, raw[u].y, sc), cvt4<DT>(raw[u].z, raw[u].w, sc));
    if (m16 > inf16<DT>()) {  // a NaN among these eight (rare)
      codes.x = nan_fix<DT>(nan_fix<DT>(codes.x, raw[u].x, 0), raw[u].y, 16);
      codes.y = nan_fix<DT>(nan_fix<DT>(codes.y, raw[u].z, 0), raw[u].w, 16);
    }
    if constexpr (PACK4) {
      const uint32_t four = gather4_stride4(biased);
      if (g < ngroups) {
        *reinterpret_cast<uint2*>(q + g * 8) = codes;
        if (scales && (threadIdx.x & 15) == 0) reinterpret_cast<uint32_t*>(scales)[g >> 4] = four;
        if (scales_km && (threadIdx.x & 3) == 0) {
          const uint32_t blocks = groups_per_row >> 2;
          const uint64_t b = g >> 2;
          const uint64_t row = b / blocks;
          scales_km[scale_pack_offset(row, b - row * blocks, (rows + 127) >> 7)] = (uint8_t)biased;
        }
      }
    } else {
      if (g < ngroups) {
        *reinterpret_cast<uint2*>(q + g * 8) = codes;
        if ((threadIdx.x & 3) == 0) scales[g >> 2] = (uint8_t)biased;
      }
    }
  }
}

// ---- cols: blocks run along the strided axis ------------------------------------------------
// Input x[r][c] (c unit stride); output q_t[c][r], scales_t[c][r/32]. A workgroup stages a
// TR x TC tile in LDS with 128-bit row loads (256-byte row segments). Then a lane owns 16 rows of
// two adjacent columns: it reads 16 dwords down the tile, joins the abs-max with the neighbouring
// lane (the other half of the 32-row block) and writes 16 bytes of each of the two q_t rows. The
// lanes that share a column pair lie side by side along the rows, so one store instruction writes
// whole contiguous 128-byte lines of q_t, not halves of them.
// Measured on [16384, 3072] bf16 against tiles of 256 x 128 with a whole block per lane (two stores
// of 16 bytes 32 bytes apart): 31.8 against 34.5 us on a ring of tensors larger than the last-level
// cache; tiles of 256 or 512 rows, 32 or 64 columns, 256 or 1024 threads and band-major or
// XCD-grouped tile orders all measure 33-36 us, and a kernel with this tile's loads and stores
// alone (no LDS, no arithmetic) 30.4 us, a sequential one 28.6. A work-group that walks two tiles down
// the rows and requests the second before it works on the first: 34.1 us; the scale bytes (four per
// q_t row and tile) cost 0.7-1.2 us of the 32.5.
constexpr int kColsThreads = 512;
constexpr int kColsTR = 128;  // rows of x per tile (4 blocks)
constexpr int kColsTC = 128;  // columns of x per tile: 256-byte row segments
constexpr int kColsPitch = kColsTC / 2 + 4;  // dwords per staged row (16-byte aligned rows)
constexpr int kColsHalves = kColsTR / 16;    // half-blocks of 16 rows per tile
constexpr int kColsSkew = 32 / kColsHalves;  // extra dwords after each 16 rows. LDS serves a 32-bit read 32 lanes and 32 banks at a time: the
                                             // 8 half-blocks x 4 column pairs of such a half-wavefront hit 32 different banks (a skew of 8, right for 64
                                             // banks, measured SQ_LDS_BANK_CONFLICT at a third of SQ_LDS_IDX_ACTIVE: two lanes per bank)

// MX: one E8M0 scale per block of 32 rows, found here. !MX: one fp32 scale per column of x (per
// row of q_t) from `col_amax`, the fp32 bits of each column's amax taken by an earlier pass;
// rows may then be any multiple of 16.
template <int DT, bool MX>
__global__ __launch_bounds__(kColsThreads) void quant_cols(
    const uint16_t* __restrict__ x, int64_t ld, int64_t rows, int64_t cols,
    uint8_t* __restrict__ q_t, uint8_t* __restrict__ scales_t, uint8_t* __restrict__ scales_km,
    const uint32_t* __restrict__ col_amax) {
  __shared__ __attribute__((aligned(16))) uint32_t tile[kColsTR * kColsPitch + kColsHalves * kColsSkew];
  const int64_t r0 = (int64_t)blockIdx.y * kColsTR;
  const int64_t c0 = (int64_t)blockIdx.x * kColsTC;
  const int tid = threadIdx.x;
  saturating_conversions();
  // stage: 16 lanes cover one 256-byte row segment
  {
    constexpr int kLanesPerRow = kColsTC / 8, kRowsPerPass = kColsThreads / kLanesPerRow, kPasses = kColsTR / kRowsPerPass;
    const int cg = tid % kLanesPerRow;  // 8-element group within the row segment
    const int rr = tid / kLanesPerRow;
    uint4 raw[kPasses];
#pragma unroll
    for (int i = 0; i < kPasses; ++i) {
      const int64_t r = r0 + rr + kRowsPerPass * i;
      const int64_t c = c0 + cg * 8;
      raw[i] = make_uint4(0, 0, 0, 0);
      if (r < rows && c < cols) raw[i] = *reinterpret_cast<const uint4*>(x + r * ld + c);
    }
#pragma unroll
    for (int i = 0; i < kPasses; ++i) {
      const int lr = rr + kRowsPerPass * i;
      *reinterpret_cast<uint4*>(&tile[lr * kColsPitch + (lr / 16) * kColsSkew + cg * 4]) = raw[i];
    }
  }
  __syncthreads();
  // lane -> (half-block of 16 rows, column pair); half-blocks vary fastest, so the 8 lanes of a column
  // pair write 128 consecutive bytes of a q_t row
  constexpr int kPairsPerTrip = kColsThreads / kColsHalves;
  static_assert((kColsTC / 2) % kPairsPerTrip == 0 && kColsHalves % 2 == 0 && kColsHalves <= 16, "lane map");
  const int h = tid % kColsHalves;
#pragma unroll
  for (int trip = 0; trip < (kColsTC / 2) / kPairsPerTrip; ++trip) {
    const int pair = tid / kColsHalves + trip * kPairsPerTrip;
    const int64_t rb = r0 + h * 16;
    const int64_t c = c0 + pair * 2;
    const uint32_t* col = &tile[h * 16 * kColsPitch + h * kColsSkew + pair];
    uint32_t w[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) w[i] = col[i * kColsPitch];
    const bool live = rb < rows && c < cols;
    uint32_t o0[4], o1[4];
    if constexpr (!MX) {
      const uint32_t ab0 = live ? col_amax[c] : 0u, ab1 = live && c + 1 < cols ? col_amax[c + 1] : 0u;
      const float s0 = scale_of_amax_bits(ab0), s1 = scale_of_amax_bits(ab1);
      const float r0 = __fdiv_rn(1.0f, s0), r1 = __fdiv_rn(1.0f, s1);
#pragma unroll
      for (int j = 0; j < 4; j += 2) {
        const uint32_t lo01 = __builtin_amdgcn_perm(w[4 * j + 1], w[4 * j], 0x05040100u), hi01 = __builtin_amdgcn_perm(w[4 * j + 1], w[4 * j], 0x07060302u);
        const uint32_t lo23 = __builtin_amdgcn_perm(w[4 * j + 3], w[4 * j + 2], 0x05040100u), hi23 = __builtin_amdgcn_perm(w[4 * j + 3], w[4 * j + 2], 0x07060302u);
        const uint32_t lo45 = __builtin_amdgcn_perm(w[4 * j + 5], w[4 * j + 4], 0x05040100u), hi45 = __builtin_amdgcn_perm(w[4 * j + 5], w[4 * j + 4], 0x07060302u);
        const uint32_t lo67 = __builtin_amdgcn_perm(w[4 * j + 7], w[4 * j + 6], 0x05040100u), hi67 = __builtin_amdgcn_perm(w[4 * j + 7], w[4 * j + 6], 0x07060302u);
        const uint2 d0 = divided_codes8<DT>(make_uint4(lo01, lo23, lo45, lo67), s0, r0, ab0 < kInfBits, ab0 > kInfBits);
        const uint2 d1 = divided_codes8<DT>(make_uint4(hi01, hi23, hi45, hi67), s1, r1, ab1 < kInfBits, ab1 > kInfBits);
        o0[j] = d0.x; o0[j + 1] = d0.y;
        o1[j] = d1.x; o1[j + 1] = d1.y;
      }
      // rows % 16 == 0: a live half-block is whole
      if (live) {
        *reinterpret_cast<uint4*>(q_t + c * rows + rb) = make_uint4(o0[0], o0[1], o0[2], o0[3]);
        if (c + 1 < cols) *reinterpret_cast<uint4*>(q_t + (c + 1) * rows + rb) = make_uint4(o1[0], o1[1], o1[2], o1[3]);
      }
    } else {
      // the two columns of the pair: low and high halves of the 16 dwords
      uint32_t mm = 0;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const v2us a = __builtin_bit_cast(v2us, w[i] & 0x7FFF7FFFu), m = __builtin_bit_cast(v2us, mm);
        mm = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(a, m));
      }
      {
        // the other half of the 32-row block is the neighbouring lane (h ^ 1): quad_perm [1,0,3,2]
        const uint32_t other = (uint32_t)__builtin_amdgcn_mov_dpp((int)mm, 0xB1, 0xF, 0xF, true);
        const v2us a = __builtin_bit_cast(v2us, other), m = __builtin_bit_cast(v2us, mm);
        mm = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(a, m));
      }
      const uint32_t m0 = mm & 0xFFFFu, m1 = mm >> 16;
      const uint32_t b0 = mx_biased_exponent(widen_bits<DT>(m0)), b1 = mx_biased_exponent(widen_bits<DT>(m1));
      const float s0 = bits_f32(b0 << 23), s1 = bits_f32(b1 << 23);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        // rows 4j .. 4j+3 of each column: regroup the halves so that a conversion sees one column
        const uint32_t lo01 = __builtin_amdgcn_perm(w[4 * j + 1], w[4 * j], 0x05040100u), hi01 = __builtin_amdgcn_perm(w[4 * j + 1], w[4 * j], 0x07060302u);
        const uint32_t lo23 = __builtin_amdgcn_perm(w[4 * j + 3], w[4 * j + 2], 0x05040100u), hi23 = __builtin_amdgcn_perm(w[4 * j + 3], w[4 * j + 2], 0x07060302u);
        o0[j] = cvt4<DT>(lo01, lo23, s0);
        o1[j] = cvt4<DT>(hi01, hi23, s1);
        if (m0 > inf16<DT>()) o0[j] = nan_fix<DT>(nan_fix<DT>(o0[j], lo01, 0), lo23, 16);
        if (m1 > inf16<DT>()) o1[j] = nan_fix<DT>(nan_fix<DT>(o1[j], hi01, 0), hi23, 16);
      }
      if (live) {
        // logical operand is [cols][rows]: row index c, block index rb / 32
        const int64_t nblk = rows / 32;
        const int64_t lb = rb / 32;
        const bool first_half = (h & 1) == 0;
        *reinterpret_cast<uint4*>(q_t + c * rows + rb) = make_uint4(o0[0], o0[1], o0[2], o0[3]);
        if (first_half) {
          if (scales_t) scales_t[c * nblk + lb] = (uint8_t)b0;
          if (scales_km) scales_km[scale_pack_offset(c, lb, (cols + 127) >> 7)] = (uint8_t)b0;
        }
        if (c + 1 < cols) {
          *reinterpret_cast<uint4*>(q_t + (c + 1) * rows + rb) = make_uint4(o1[0], o1[1], o1[2], o1[3]);
          if (first_half) {
            if (scales_t) scales_t[(c + 1) * nblk + lb] = (uint8_t)b1;
            if (scales_km) scales_km[scale_pack_offset(c + 1, lb, (cols + 127) >> 7)] = (uint8_t)b1;
          }
        }
      }
    }
  }
}

// fp32 bits of the abs-max of every column of a row-major [rows][cols] matrix, merged into
// `col_amax` (zeroed beforehand) with one atomic max per column and workgroup. Tiles as above.
__global__ void fill_u32_n(uint32_t* p, int64_t n, uint32_t v) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = v;
}

constexpr int kAmaxTR = 256, kAmaxTC = 128;  // tile of the column abs-max pass
template <int DT>
__global__ __launch_bounds__(kColsThreads) void cols_amax(const uint16_t* __restrict__ x, int64_t ld, int64_t rows,
                                                          int64_t cols, uint32_t* __restrict__ col_amax) {
  constexpr int kLanesPerRow = kAmaxTC / 8, kRowGroups = kColsThreads / kLanesPerRow;
  __shared__ uint32_t part[kRowGroups][kAmaxTC / 2 + 1];
  const int64_t r0 = (int64_t)blockIdx.y * kAmaxTR;
  const int64_t c0 = (int64_t)blockIdx.x * kAmaxTC;
  const int cg = threadIdx.x % kLanesPerRow, rr = threadIdx.x / kLanesPerRow;
  const int64_t c = c0 + cg * 8;
  uint4 raw[kAmaxTR / kRowGroups];
#pragma unroll
  for (int i = 0; i < kAmaxTR / kRowGroups; ++i) {
    const int64_t r = r0 + rr + kRowGroups * i;
    raw[i] = make_uint4(0, 0, 0, 0);
    if (r < rows && c < cols) raw[i] = *reinterpret_cast<const uint4*>(x + r * ld + c);
  }
  v2us m[4] = {{0, 0}, {0, 0}, {0, 0}, {0, 0}};
#pragma unroll
  for (int i = 0; i < kAmaxTR / kRowGroups; ++i) {
    const uint32_t w[4] = {raw[i].x, raw[i].y, raw[i].z, raw[i].w};
#pragma unroll
    for (int k = 0; k < 4; ++k) m[k] = __builtin_elementwise_max(m[k], __builtin_bit_cast(v2us, w[k] & 0x7FFF7FFFu));
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) part[rr][cg * 4 + k] = __builtin_bit_cast(uint32_t, m[k]);
  __syncthreads();
  if (threadIdx.x < kAmaxTC / 2) {
    v2us a = {0, 0};
#pragma unroll 8
    for (int g = 0; g < kRowGroups; ++g) a = __builtin_elementwise_max(a, __builtin_bit_cast(v2us, part[g][threadIdx.x]));
    const int64_t cc = c0 + threadIdx.x * 2;
    if (cc < cols && a.x != 0) atomicMax(col_amax + cc, widen_bits<DT>(a.x));
    if (cc + 1 < cols && a.y != 0) atomicMax(col_amax + cc + 1, widen_bits<DT>(a.y));
  }
}

__global__ void amax_bits_to_scales(uint32_t* p, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = f32_bits(scale_of_amax_bits(p[i]));
}

// ---- generic: any strides, one thread per block ----------------------------------------------
template <int DT>
__global__ __launch_bounds__(256) void quant_mx_generic(
    const uint16_t* __restrict__ x, int64_t sr, int64_t sc, int64_t rows, int64_t cols,
    uint8_t* __restrict__ q, uint8_t* __restrict__ scales, uint8_t* __restrict__ scales_km) {
  const int64_t nblk = cols / 32;
  const int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (b >= rows * nblk) return;
  const int64_t r = b / nblk, cb = b - r * nblk;
  const uint16_t* src = x + r * sr + cb * 32 * sc;
  float f[32];
  uint32_t m = 0;
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    f[i] = widen<DT>(src[i * sc]);
    const uint32_t a = f32_bits(f[i]) & kAbsMask;
    m = a > m ? a : m;
  }
  const uint32_t biased = mx_biased_exponent(m);
  const float inv = mx_inverse_scale(biased);
  uint8_t* dst = q + r * cols + cb * 32;
#pragma unroll
  for (int i = 0; i < 32; ++i) dst[i] = (uint8_t)e4m3_encode(f[i] * inv);
  if (scales) scales[b] = (uint8_t)biased;
  if (scales_km) scales_km[scale_pack_offset(r, cb, (rows + 127) >> 7)] = (uint8_t)biased;
}

// natural scales [rows, blocks] -> MFMA-packed; one byte per thread
__global__ __launch_bounds__(256) void scales_pack(const uint8_t* __restrict__ in, int64_t rows, int64_t blocks,
                                                   uint8_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= rows * blocks) return;
  const int64_t r = i / blocks, b = i - r * blocks;
  out[scale_pack_offset(r, b, (rows + 127) >> 7)] = in[i];
}

// ---- per-tensor recipe -----------------------------------------------------------------------

// The abs-max pass leaves one partial maximum per work-group in the call's workspace and the cast pass
// reduces them again in every work-group (at most 512 words, from L2, under its first loads): no word
// to clear beforehand, so no launch for that, and no atomics. Atomics on one address are served one at a
// time, about 10 ns each, while the wavefronts that issued them keep their slots: 2048 work-groups of 256
// threads cost 19 us in atomics on top of 16 us of reading; even 512 that first look at the value and skip
// the atomic when it cannot raise it end in a queue, because they all finish at once. The pass runs few,
// large work-groups (two per compute unit, 1024 threads, four 128-bit loads in flight per thread and the
// next four requested before these are looked at).
// (A single launch that reads the tensor once, keeps it in registers across a grid-wide wait and converts
// from there was built and measured: 46 us against 44 us for the two passes on [16384, 3072]. Its loads
// and its stores are separate phases, 32 us even without the wait and the arithmetic, where a streaming
// kernel overlaps them; the second pass here reads from the last-level cache anyway.)
constexpr int kAmaxThreads = 1024;
constexpr int kAmaxBlocks = 512;
static_assert(kAmaxBlocks * 4 <= KM_QUANT_TENSOR_WORKSPACE_BYTES, "one partial maximum per work-group of the abs-max pass");
constexpr int kAmaxPiece = kAmaxThreads * 4;  // 128-bit chunks per work-group and trip (64 KiB)
constexpr int kTensorBlocks = 1 << 20;        // the cast pass: one 16 KiB piece per work-group, grid-stride beyond

// non-negative floats order like their bits: an unsigned max of fp32 bits is an abs-max
// (NaN patterns stay above infinity). partials[blockIdx.x] = this work-group's maximum.
template <int DT>
__global__ __launch_bounds__(kAmaxThreads) void tensor_amax(const uint16_t* __restrict__ x, int64_t sr,
                                                            int64_t sc, int64_t rows, int64_t cols,
                                                            uint32_t* __restrict__ partials) {
  constexpr int T = kAmaxThreads;
  const int64_t n = rows * cols;
  const bool dense = sc == 1 && sr == cols;
  uint32_t m16 = 0;
  if (dense && (cols % 8) == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0) {
    // a work-group reads whole pieces (four consecutive runs of 16 KiB, one per load of a thread)
    const uint4* src = reinterpret_cast<const uint4*>(x);
    const int64_t nch = n / 8;
    const int64_t first = (int64_t)blockIdx.x * kAmaxPiece, hop = (int64_t)gridDim.x * kAmaxPiece;
    auto take = [&](const uint4 (&r)[4]) __attribute__((always_inline)) {
      const uint32_t a = amax16x8(r[0]), b = amax16x8(r[1]), c = amax16x8(r[2]), d = amax16x8(r[3]);
      const uint32_t ab = a > b ? a : b, cd = c > d ? c : d, abcd = ab > cd ? ab : cd;
      m16 = abcd > m16 ? abcd : m16;
    };
    // whole pieces, the loads of the next one issued before this one is looked at: a work-group that
    // waits for a piece, reduces it and only then asks for the next leaves the memory system idle in between
    int64_t base = first;
    uint4 cur[4], nxt[4];
    bool have = base + kAmaxPiece <= nch;
    if (have) {
#pragma unroll
      for (int i = 0; i < 4; ++i) cur[i] = src[base + threadIdx.x + i * T];
    }
    while (have) {
      const int64_t after = base + hop;
      const bool more = after + kAmaxPiece <= nch;
      if (more) {
#pragma unroll
        for (int i = 0; i < 4; ++i) nxt[i] = src[after + threadIdx.x + i * T];
      }
      take(cur);
#pragma unroll
      for (int i = 0; i < 4; ++i) cur[i] = nxt[i];
      base = after;
      have = more;
    }
    // the ragged last piece belongs to the work-group whose walk reaches it
    if (base < nch) {
      for (int64_t i = base + threadIdx.x; i < nch; i += T) {
        const uint32_t a = amax16x8(src[i]);
        m16 = a > m16 ? a : m16;
      }
    }
  } else {
    const int64_t stride = (int64_t)gridDim.x * T;
    for (int64_t i = (int64_t)blockIdx.x * T + threadIdx.x; i < n; i += stride) {
      const int64_t r = i / cols, c = i - r * cols;
      const uint32_t a = x[r * sr + c * sc] & 0x7FFFu;
      m16 = a > m16 ? a : m16;
    }
  }
  __shared__ uint32_t wave_m[T / 64];
  const uint32_t m = wave_max(m16);
  if ((threadIdx.x & 63) == 0) wave_m[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x < 64) {
    const uint32_t mine = threadIdx.x < T / 64 ? wave_m[threadIdx.x] : 0u;
    const uint32_t bits = widen_bits<DT>(wave_max(mine));
    if (threadIdx.x == 0) partials[blockIdx.x] = bits;
  }
}

template <int DT>
__global__ __launch_bounds__(256) void tensor_cast(const uint16_t* __restrict__ x, int64_t sr,
                                                   int64_t sc, int64_t rows, int64_t cols,
                                                   const uint32_t* __restrict__ partials, int npartials,
                                                   uint8_t* __restrict__ q,
                                                   float* __restrict__ scale_out) {
  saturating_conversions();
  // the tensor's abs-max: every work-group reduces the abs-max pass's partial maxima (npartials <= 512)
  __shared__ uint32_t wave_m[4];
  uint32_t mine = 0;
  for (int i = threadIdx.x; i < npartials; i += 256) {
    const uint32_t v = partials[i];
    mine = v > mine ? v : mine;
  }
  mine = wave_max(mine);
  if ((threadIdx.x & 63) == 0) wave_m[threadIdx.x >> 6] = mine;
  __syncthreads();
  const uint32_t ab01 = wave_m[0] > wave_m[1] ? wave_m[0] : wave_m[1], ab23 = wave_m[2] > wave_m[3] ? wave_m[2] : wave_m[3];
  const uint32_t ab = ab01 > ab23 ? ab01 : ab23;
  const bool finite = ab < kInfBits, nan_all = ab > kInfBits;
  const float s = nan_all ? bits_f32(0x7FC00000u) : __fdiv_rn(bits_f32(ab > kAmaxFloorBits ? ab : kAmaxFloorBits), 448.0f);
  const float rcp = __fdiv_rn(1.0f, s);
  if (blockIdx.x == 0 && threadIdx.x == 0 && scale_out) *scale_out = s;
  const int64_t n = rows * cols;
  const bool dense = sc == 1 && sr == cols;
  const int64_t stride = (int64_t)gridDim.x * 256;
  if (dense && (cols % 8) == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0) {
    const uint4* src = reinterpret_cast<const uint4*>(x);
    uint2* dst = reinterpret_cast<uint2*>(q);
    const int64_t nch = n / 8;
    // whole 16 KiB pieces per work-group, as in the abs-max pass
    for (int64_t base = (int64_t)blockIdx.x * 1024; base < nch; base += (int64_t)gridDim.x * 1024) {
      const int64_t g = base + threadIdx.x;
      if (base + 1024 <= nch) {
        const uint4 r0 = src[g], r1 = src[g + 256], r2 = src[g + 512], r3 = src[g + 768];
        dst[g] = divided_codes8<DT>(r0, s, rcp, finite, nan_all);
        dst[g + 256] = divided_codes8<DT>(r1, s, rcp, finite, nan_all);
        dst[g + 512] = divided_codes8<DT>(r2, s, rcp, finite, nan_all);
        dst[g + 768] = divided_codes8<DT>(r3, s, rcp, finite, nan_all);
      } else {
        for (int64_t i = g; i < nch; i += 256) dst[i] = divided_codes8<DT>(src[i], s, rcp, finite, nan_all);
      }
    }
  } else {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
      const int64_t r = i / cols, c = i - r * cols;
      q[i] = (uint8_t)divided_code1<DT>(x[r * sr + c * sc], s, finite, nan_all);
    }
  }
}

// ---- per-row recipe: one wavefront per row -----------------------------------------------------
constexpr int kRowRecipeHeld = 8;  // 128-bit loads a lane keeps in registers: rows up to 4096 elements are read once

// Unit-stride rows, cols = 8 * chunks. HELD: the whole row stays in registers between the
// amax pass and the conversion; otherwise the second pass reads it again (from L2: a wavefront
// re-reads what it has just fetched).
template <int DT, bool HELD>
__global__ __launch_bounds__(256) void quant_fp8_rows(const uint16_t* __restrict__ x, int64_t ld, uint32_t chunks,
                                                      uint32_t rows, uint8_t* __restrict__ q, float* __restrict__ scale) {
  saturating_conversions();
  const uint32_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
  const uint32_t lane = threadIdx.x & 63;
  if (row >= rows) return;
  const uint4* src = reinterpret_cast<const uint4*>(x + (uint64_t)row * (uint64_t)ld);
  uint2* dst = reinterpret_cast<uint2*>(q + (uint64_t)row * chunks * 8);
  uint4 raw[HELD ? kRowRecipeHeld : 1];
  uint32_t m16 = 0;
  if constexpr (HELD) {
#pragma unroll
    for (int u = 0; u < kRowRecipeHeld; ++u) {
      const uint32_t c = lane + 64 * u;
      raw[u] = c < chunks ? src[c] : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int u = 0; u < kRowRecipeHeld; ++u) {
      const uint32_t a = amax16x8(raw[u]);
      m16 = a > m16 ? a : m16;
    }
  } else {
    for (uint32_t c = lane; c < chunks; c += 64) {
      const uint32_t a = amax16x8(src[c]);
      m16 = a > m16 ? a : m16;
    }
  }
  m16 = wave_max(m16);
  const float s = scale_of_amax16<DT>(m16);
  const float rcp = __fdiv_rn(1.0f, s);
  if (lane == 0) scale[row] = s;
  const bool finite = m16 < inf16<DT>(), nan_row = m16 > inf16<DT>();
  if constexpr (HELD) {
#pragma unroll
    for (int u = 0; u < kRowRecipeHeld; ++u) {
      const uint32_t c = lane + 64 * u;
      if (c < chunks) dst[c] = divided_codes8<DT>(raw[u], s, rcp, finite, nan_row);
    }
  } else {
    for (uint32_t c = lane; c < chunks; c += 64) dst[c] = divided_codes8<DT>(src[c], s, rcp, finite, nan_row);
  }
}

// Any strides and lengths: one wavefront per row, one element per lane and trip.
template <int DT>
__global__ __launch_bounds__(256) void quant_fp8_rows_generic(const uint16_t* __restrict__ x, int64_t sr, int64_t sc,
                                                              uint32_t rows, int64_t cols, uint8_t* __restrict__ q,
                                                              float* __restrict__ scale) {
  saturating_conversions();
  const uint32_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
  const uint32_t lane = threadIdx.x & 63;
  if (row >= rows) return;
  const uint16_t* src = x + (int64_t)row * sr;
  uint32_t m16 = 0;
  for (int64_t c = lane; c < cols; c += 64) {
    const uint32_t a = src[c * sc] & 0x7FFFu;
    m16 = a > m16 ? a : m16;
  }
  m16 = wave_max(m16);
  const float s = scale_of_amax16<DT>(m16);
  if (lane == 0) scale[row] = s;
  const bool finite = m16 < inf16<DT>(), nan_row = m16 > inf16<DT>();
  uint8_t* dst = q + (int64_t)row * cols;
  for (int64_t c = lane; c < cols; c += 64) {
    dst[c] = (uint8_t)divided_code1<DT>(src[c * sc], s, finite, nan_row);
  }
}

// ---- int8 per-row quantizer ----------------------------------------------------------------------
// s[r] = max(amax_r, 1e-12) / 127 and q = clamp(round_half_even(x / s[r]), +-127), IEEE fp32
// divisions, the columns multiplied by `col_scale` first (in fp32) when given (reference
// src/kohakumoss_kernels/int8/formats.py:21-38; Triton backends/triton/int8.py). One wavefront
// per row; NaN inputs are outside the contract (the reference's cast of NaN to int8 is
// platform-defined).
__device__ __forceinline__ uint32_t i8_code(float v, float s) {
  const float r = __builtin_amdgcn_fmed3f(__builtin_rintf(__fdiv_rn(v, s)), -127.0f, 127.0f);
  return (uint32_t)(int)r & 0xFFu;
}

template <int DT>
__device__ __forceinline__ void scaled8(const uint4& raw, const float* __restrict__ col_scale, uint32_t chunk, float (&f)[8]) {
  widen8<DT>(raw, f);
  if (col_scale != nullptr) {
    const float4 c0 = reinterpret_cast<const float4*>(col_scale)[2 * chunk], c1 = reinterpret_cast<const float4*>(col_scale)[2 * chunk + 1];
    f[0] *= c0.x; f[1] *= c0.y; f[2] *= c0.z; f[3] *= c0.w;
    f[4] *= c1.x; f[5] *= c1.y; f[6] *= c1.z; f[7] *= c1.w;
  }
}

__device__ __forceinline__ uint32_t amax_bits_of8(const float (&f)[8]) {
  uint32_t m = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t a = f32_bits(f[i]) & kAbsMask;
    m = a > m ? a : m;
  }
  return m;
}

__device__ __forceinline__ float i8_scale_of(uint32_t amax_bits) {
  return __fdiv_rn(bits_f32(amax_bits > kAmaxFloorBits ? amax_bits : kAmaxFloorBits), 127.0f);
}

template <int DT, bool HELD>
__global__ __launch_bounds__(256) void quant_i8_rows(const uint16_t* __restrict__ x, int64_t ld, uint32_t chunks, uint32_t rows,
                                                     const float* __restrict__ col_scale, uint8_t* __restrict__ q,
                                                     float* __restrict__ scale) {
  const uint32_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
  const uint32_t lane = threadIdx.x & 63;
  if (row >= rows) return;
  const uint4* src = reinterpret_cast<const uint4*>(x + (uint64_t)row * (uint64_t)ld);
  uint2* dst = reinterpret_cast<uint2*>(q + (uint64_t)row * chunks * 8);
  uint4 raw[HELD ? kRowRecipeHeld : 1];
  uint32_t m = 0;
  float f[8];
  if constexpr (HELD) {
#pragma unroll
    for (int u = 0; u < kRowRecipeHeld; ++u) {
      const uint32_t c = lane + 64 * u;
      raw[u] = c < chunks ? src[c] : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int u = 0; u < kRowRecipeHeld; ++u) {
      const uint32_t c = lane + 64 * u;
      if (c < chunks) {
        scaled8<DT>(raw[u], col_scale, c, f);
        const uint32_t a = amax_bits_of8(f);
        m = a > m ? a : m;
      }
    }
  } else {
    for (uint32_t c = lane; c < chunks; c += 64) {
      scaled8<DT>(src[c], col_scale, c, f);
      const uint32_t a = amax_bits_of8(f);
      m = a > m ? a : m;
    }
  }
  m = wave_max(m);
  const float s = i8_scale_of(m);
  if (lane == 0) scale[row] = s;
  // Without column scales the inputs are 16-bit patterns below the row's amax: the quotient then
  // comes from the rounded reciprocal and two fused corrections, as in the fp8 row quantizer (equal
  // to the division wherever the rounded quotient is not zero; the GPU tests compare every (amax, x)
  // pair with the dividing element-wise kernel). Column-scaled inputs are arbitrary fp32 values and a
  // row with an infinite amax follows the division's special cases: both divide.
  const bool fast = col_scale == nullptr && m < kInfBits;
  const float rcp = __fdiv_rn(1.0f, s);
  auto codes = [&](const uint4& r, uint32_t c) __attribute__((always_inline)) {
    scaled8<DT>(r, col_scale, c, f);
    uint32_t b[8];
    if (fast) {
#pragma unroll
      for (int i = 0; i < 8; ++i) b[i] = (uint32_t)(int)__builtin_amdgcn_fmed3f(__builtin_rintf(quotient(f[i], s, rcp)), -127.0f, 127.0f) & 0xFFu;
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) b[i] = i8_code(f[i], s);
    }
    return make_uint2(b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24), b[4] | (b[5] << 8) | (b[6] << 16) | (b[7] << 24));
  };
  if constexpr (HELD) {
#pragma unroll
    for (int u = 0; u < kRowRecipeHeld; ++u) {
      const uint32_t c = lane + 64 * u;
      if (c < chunks) dst[c] = codes(raw[u], c);
    }
  } else {
    for (uint32_t c = lane; c < chunks; c += 64) dst[c] = codes(src[c], c);
  }
}

template <int DT>
__global__ __launch_bounds__(256) void quant_i8_rows_generic(const uint16_t* __restrict__ x, int64_t sr, int64_t sc, uint32_t rows,
                                                             int64_t cols, const float* __restrict__ col_scale,
                                                             uint8_t* __restrict__ q, float* __restrict__ scale) {
  const uint32_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
  const uint32_t lane = threadIdx.x & 63;
  if (row >= rows) return;
  const uint16_t* src = x + (int64_t)row * sr;
  uint32_t m = 0;
  for (int64_t c = lane; c < cols; c += 64) {
    float v = widen<DT>(src[c * sc]);
    if (col_scale != nullptr) v *= col_scale[c];
    const uint32_t a = f32_bits(v) & kAbsMask;
    m = a > m ? a : m;
  }
  m = wave_max(m);
  const float s = i8_scale_of(m);
  if (lane == 0) scale[row] = s;
  uint8_t* dst = q + (int64_t)row * cols;
  for (int64_t c = lane; c < cols; c += 64) {
    float v = widen<DT>(src[c * sc]);
    if (col_scale != nullptr) v *= col_scale[c];
    dst[c] = (uint8_t)i8_code(v, s);
  }
}

// ---- int8 per-row quantizer of a rotated activation ---------------------------------------------
// q, s = quantize_rows(group_hadamard(x, G)) in one pass over x (the reference's Triton quantizer
// rotates the tile it has loaded, backends/triton/int8.py:47-75). A work-group owns one row of up to
// 4096 elements: it widens the row into LDS and runs the butterfly stages of km_hadamard.hip there
// (same stages, same order, the same rounding to the 16-bit type at the end: the rotated values are
// those the rotation kernel would have written). The last double pass leaves a lane with 16
// consecutive rotated elements in registers; the row's abs-max is joined over the work-group and the
// lane writes its 16 codes with one 128-bit store: the rotated row never goes back to LDS or memory.
// Groups of 16 and more (a group of 4 has no double pass; it takes the two kernels).
constexpr int kRotMaxCols = 4096;

template <int DT, int J>
__global__ __launch_bounds__(256) void rotate_quant_i8_rows(const uint16_t* __restrict__ x, int64_t ld, uint32_t cols,
                                                            uint8_t* __restrict__ q, float* __restrict__ scale) {
  static_assert(J >= 2, "the last stages run as a double pass");
  constexpr int G = 1 << (2 * J);
  constexpr float kScale = 1.0f / (float)(1 << J);
  __shared__ __attribute__((aligned(16))) float tile[kRotMaxCols];
  __shared__ uint32_t wave_m[4];
  const uint32_t t = threadIdx.x, row = blockIdx.x;
  const uint32_t chunks = cols / 8, units = cols / 16;
  const uint4* src = reinterpret_cast<const uint4*>(x + (uint64_t)row * (uint64_t)ld);
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const uint32_t c = t + 256 * i;
    if (c < chunks) {
      float f[8];
      widen8<DT>(src[c], f);
      *reinterpret_cast<float4*>(&tile[c * 8]) = make_float4(f[0], f[1], f[2], f[3]);
      *reinterpret_cast<float4*>(&tile[c * 8 + 4]) = make_float4(f[4], f[5], f[6], f[7]);
    }
  }
  __syncthreads();
  if constexpr (J % 2 == 1) {
    constexpr uint32_t S1 = G / 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t qd = t + 256 * i;
      if (qd < cols / 4) {
        const uint32_t first = (qd / S1) * 4 * S1 + qd % S1;
        float v0 = tile[first], v1 = tile[first + S1], v2 = tile[first + 2 * S1], v3 = tile[first + 3 * S1];
        h4(v0, v1, v2, v3);
        tile[first] = v0; tile[first + S1] = v1; tile[first + 2 * S1] = v2; tile[first + 3 * S1] = v3;
      }
    }
    __syncthreads();
  }
  constexpr int kDouble = J / 2;
  constexpr uint32_t kRest = J % 2 == 1 ? G / 4 : G;
  float v[4][4];
  const bool active = t < units;
#pragma unroll
  for (int p = 0; p < kDouble; ++p) {
    const uint32_t S = kRest >> (4 * (p + 1));
    const uint32_t first = (t / S) * 16 * S + t % S;
    if (active) {
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) v[a][b] = tile[first + (4 * a + b) * S];
#pragma unroll
      for (int b = 0; b < 4; ++b) h4(v[0][b], v[1][b], v[2][b], v[3][b]);
#pragma unroll
      for (int a = 0; a < 4; ++a) h4(v[a][0], v[a][1], v[a][2], v[a][3]);
    }
    if (p < kDouble - 1) {
      if (active) {
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
          for (int b = 0; b < 4; ++b) tile[first + (4 * a + b) * S] = v[a][b];
      }
      __syncthreads();
    }
  }
  // lane t holds elements [16 t, 16 t + 16) of the rotated row: round them as the rotation kernel
  // stores them, join the abs-max, quantize
  uint32_t m = 0;
  if (active) {
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        v[a][b] = had_widen<DT>(had_narrow<DT>(v[a][b] * kScale));
        const uint32_t bits = f32_bits(v[a][b]) & kAbsMask;
        m = bits > m ? bits : m;
      }
  }
  m = wave_max(m);
  if ((t & 63) == 0) wave_m[t >> 6] = m;
  __syncthreads();
  {
    const uint32_t m01 = wave_m[0] > wave_m[1] ? wave_m[0] : wave_m[1], m23 = wave_m[2] > wave_m[3] ? wave_m[2] : wave_m[3];
    m = m01 > m23 ? m01 : m23;
  }
  const float s = i8_scale_of(m);
  if (t == 0) scale[row] = s;
  if (!active) return;
  // the rotated values are 16-bit patterns at or below the row's amax: the quotient comes from the
  // rounded reciprocal and two fused corrections, as in quant_i8_rows; a row with an infinite amax divides
  const bool fast = m < kInfBits;
  const float rcp = __fdiv_rn(1.0f, s);
  uint32_t packed[4];
#pragma unroll
  for (int a = 0; a < 4; ++a) {
    uint32_t b4[4];
#pragma unroll
    for (int b = 0; b < 4; ++b)
      b4[b] = fast ? ((uint32_t)(int)__builtin_amdgcn_fmed3f(__builtin_rintf(quotient(v[a][b], s, rcp)), -127.0f, 127.0f) & 0xFFu) : i8_code(v[a][b], s);
    packed[a] = b4[0] | (b4[1] << 8) | (b4[2] << 16) | (b4[3] << 24);
  }
  *reinterpret_cast<uint4*>(q + (uint64_t)row * cols + 16 * t) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
}

// ---- block recipe: fp32 scales per 128 columns (activations) or per 128 x 128 block (weights) ----
// s = max(amax, 1e-12) / 448 and q = e4m3(clamp(x / s)) as in the per-row recipe, over smaller
// groups (reference src/kohakumoss_kernels/fp8/formats.py:83-93).

// max over the 16 lanes of a DPP row, in every lane of the row
__device__ __forceinline__ uint32_t row16_max(uint32_t v) {
  v = quad_max(v);
  uint32_t o = (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x124, 0xF, 0xF, true);  // row_ror:4
  v = v > o ? v : o;
  o = (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x128, 0xF, 0xF, true);  // row_ror:8
  return v > o ? v : o;
}

// Activations, unit-stride rows: lane = 8 consecutive elements, 16 lanes = one block of 128.
// q and the scales [rows, cols/128] are contiguous, so both are indexed by the flat group number.
template <int DT>
__global__ __launch_bounds__(kRowsThreads) void quant_fp8_blocks_act(const uint16_t* __restrict__ x, int64_t ld, uint32_t groups_per_row,
                                                                     uint64_t ngroups, uint32_t rows, uint8_t* __restrict__ q, float* __restrict__ scale,
                                                                     float* __restrict__ scale_km) {
  saturating_conversions();
  const uint64_t base = (uint64_t)blockIdx.x * (kRowsThreads * kRowsUnroll) + threadIdx.x;
  const bool dense = ld == (int64_t)groups_per_row * 8;
  uint4 raw[kRowsUnroll];
#pragma unroll
  for (int u = 0; u < kRowsUnroll; ++u) {
    const uint64_t g = base + (uint64_t)u * kRowsThreads;
    raw[u] = make_uint4(0, 0, 0, 0);
    if (g < ngroups) {
      uint64_t off;
      if (dense) {
        off = g * 8;
      } else {
        const uint64_t row = g / groups_per_row;
        off = row * (uint64_t)ld + (g - row * groups_per_row) * 8;
      }
      raw[u] = *reinterpret_cast<const uint4*>(x + off);
    }
  }
#pragma unroll
  for (int u = 0; u < kRowsUnroll; ++u) {
    const uint64_t g = base + (uint64_t)u * kRowsThreads;
    const uint32_t m16 = row16_max(amax16x8(raw[u]));
    const float s = scale_of_amax16<DT>(m16);
    const float rcp = __fdiv_rn(1.0f, s);
    const uint2 codes = divided_codes8<DT>(raw[u], s, rcp, m16 < inf16<DT>(), m16 > inf16<DT>());
    if (g < ngroups) {
      *reinterpret_cast<uint2*>(q + g * 8) = codes;
      if ((threadIdx.x & 15) == 0) {
        if (scale) scale[g >> 4] = s;
        if (scale_km) {  // [cols/128, rows]: the layout the GEMM reads with one run per 16 rows
          const uint32_t blocks = groups_per_row >> 4;
          const uint64_t b = g >> 4, row = b / blocks;
          scale_km[(b - row * blocks) * rows + row] = s;
        }
      }
    }
  }
}

// Weights, unit-stride rows: a workgroup owns one 128 x 128 block, held in registers (eight
// 128-bit loads per lane) between the amax pass and the conversion. Rows past the end count as zeros.
template <int DT>
__global__ __launch_bounds__(256) void quant_fp8_blocks_weight(const uint16_t* __restrict__ x, int64_t ld, int64_t rows, int64_t cols,
                                                               uint8_t* __restrict__ q, float* __restrict__ scale) {
  saturating_conversions();
  __shared__ uint32_t wave_amax[4];
  const int64_t r0 = (int64_t)blockIdx.y * 128, c0 = (int64_t)blockIdx.x * 128;
  const int chunk = threadIdx.x & 15, rsub = threadIdx.x >> 4;
  uint4 raw[8];
  uint32_t m16 = 0;
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const int64_t r = r0 + rsub + 16 * u;
    raw[u] = r < rows ? *reinterpret_cast<const uint4*>(x + r * ld + c0 + chunk * 8) : make_uint4(0, 0, 0, 0);
  }
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const uint32_t a = amax16x8(raw[u]);
    m16 = a > m16 ? a : m16;
  }
  m16 = wave_max(m16);
  if ((threadIdx.x & 63) == 0) wave_amax[threadIdx.x >> 6] = m16;
  __syncthreads();
  m16 = max(max(wave_amax[0], wave_amax[1]), max(wave_amax[2], wave_amax[3]));
  const float s = scale_of_amax16<DT>(m16);
  const float rcp = __fdiv_rn(1.0f, s);
  if (threadIdx.x == 0) scale[(int64_t)blockIdx.y * gridDim.x + blockIdx.x] = s;
  const bool finite = m16 < inf16<DT>(), nan_block = m16 > inf16<DT>();
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const int64_t r = r0 + rsub + 16 * u;
    if (r < rows) *reinterpret_cast<uint2*>(q + r * cols + c0 + chunk * 8) = divided_codes8<DT>(raw[u], s, rcp, finite, nan_block);
  }
}

// Any strides: a workgroup per 128 x 128 tile, two lanes per row of the tile (64 elements each),
// dividing element by element. WEIGHT: one scale for the tile, else one per row of the tile (and
// its [cols/128, rows] copy when asked for).
// A transposed view (stride_row == 1) still reads neighbouring rows with neighbouring lanes.
template <int DT, bool WEIGHT>
__global__ __launch_bounds__(256) void quant_fp8_blocks_generic(const uint16_t* __restrict__ x, int64_t sr, int64_t sc, int64_t rows,
                                                                int64_t cols, uint8_t* __restrict__ q, float* __restrict__ scale,
                                                                float* __restrict__ scale_km) {
  saturating_conversions();
  __shared__ uint32_t wave_amax[4];
  const int64_t r = (int64_t)blockIdx.y * 128 + (threadIdx.x >> 1);
  const int64_t c0 = (int64_t)blockIdx.x * 128 + (threadIdx.x & 1) * 64;
  const bool live = r < rows;
  const uint16_t* src = x + r * sr + c0 * sc;
  uint32_t m16 = 0;
  if (live) {
    for (int c = 0; c < 64; ++c) {
      const uint32_t a = src[c * sc] & 0x7FFFu;
      m16 = a > m16 ? a : m16;
    }
  }
  if constexpr (WEIGHT) {
    m16 = wave_max(m16);
    if ((threadIdx.x & 63) == 0) wave_amax[threadIdx.x >> 6] = m16;
    __syncthreads();
    m16 = max(max(wave_amax[0], wave_amax[1]), max(wave_amax[2], wave_amax[3]));
  } else {
    const uint32_t o = (uint32_t)__shfl_xor((int)m16, 1);
    m16 = o > m16 ? o : m16;
  }
  const float s = scale_of_amax16<DT>(m16);
  if constexpr (WEIGHT) {
    if (threadIdx.x == 0) scale[(int64_t)blockIdx.y * gridDim.x + blockIdx.x] = s;
  } else {
    if (live && (threadIdx.x & 1) == 0) {
      if (scale) scale[r * gridDim.x + blockIdx.x] = s;
      if (scale_km) scale_km[(int64_t)blockIdx.x * rows + r] = s;
    }
  }
  if (!live) return;
  const bool finite = m16 < inf16<DT>(), nan_block = m16 > inf16<DT>();
  uint8_t* dst = q + r * cols + c0;
  for (int c = 0; c < 64; ++c) dst[c] = (uint8_t)divided_code1<DT>(src[c * sc], s, finite, nan_block);
}

}  // namespace km

using namespace km;

#define KM_DISPATCH_DT(dt, ...)                       \
  if ((dt) == KM_BF16) {                              \
    constexpr int DT = KM_BF16;                       \
    __VA_ARGS__;                                      \
  } else {                                            \
    constexpr int DT = KM_F16;                        \
    __VA_ARGS__;                                      \
  }

extern "C" int km_quant_mx(const void* x, int64_t rows, int64_t cols, int64_t stride_row,
                           int64_t stride_col, int dtype, void* q, void* scales, void* scales_packed,
                           void* stream) {
  if (dtype != KM_BF16 && dtype != KM_F16) return km_fail(KM_ERR_ARG, "km_quant_mx: dtype must be bf16 or f16");
  if (rows < 0 || cols < 0 || cols % 32) return km_fail(KM_ERR_ARG, "km_quant_mx: cols must be a non-negative multiple of 32");
  if (scales_packed && cols % 128) return km_fail(KM_ERR_ARG, "km_quant_mx: the packed scale copy needs cols % 128 == 0");
  if (rows == 0 || cols == 0) return KM_OK;
  if (!x || !q || (!scales && !scales_packed)) return km_fail(KM_ERR_ARG, "km_quant_mx: null pointer");
  if (reinterpret_cast<uintptr_t>(scales) & 3) return km_fail(KM_ERR_ARG, "km_quant_mx: scales must be 4-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  const uint16_t* xp = (const uint16_t*)x;
  uint8_t *qp = (uint8_t*)q, *sp = (uint8_t*)scales, *kp = (uint8_t*)scales_packed;
  const bool aligned = (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(q) & 15) == 0;
  const uint64_t ngroups = (uint64_t)rows * (uint64_t)cols / 8;
  if (stride_col == 1 && aligned && stride_row % 8 == 0 && stride_row >= cols && ngroups < (1ull << 40) && rows < (1ll << 31)) {
    const uint64_t per_block = (uint64_t)kRowsThreads * kRowsUnroll;
    const uint64_t blocks = (ngroups + per_block - 1) / per_block;
    if (blocks > 0x7FFFFFFFull) return km_fail(KM_ERR_ARG, "km_quant_mx: tensor too large");
    const bool pack4 = cols % 128 == 0;
    if (!pack4 && !sp) return km_fail(KM_ERR_ARG, "km_quant_mx: null scales");
    KM_DISPATCH_DT(dtype, {
      if (pack4)
        hipLaunchKernelGGL((quant_mx_rows<DT, true>), dim3((unsigned)blocks), dim3(kRowsThreads), 0, st, xp, stride_row,
                           (uint32_t)(cols / 8), ngroups, (uint32_t)rows, qp, sp, kp);
      else
        hipLaunchKernelGGL((quant_mx_rows<DT, false>), dim3((unsigned)blocks), dim3(kRowsThreads), 0, st, xp, stride_row,
                           (uint32_t)(cols / 8), ngroups, (uint32_t)rows, qp, sp, kp);
    });
  } else if (stride_row == 1 && aligned && stride_col % 8 == 0 && stride_col >= rows && rows % 8 == 0) {
    // the memory is a row-major [cols][rows] matrix read along its unit-stride axis; blocks of
    // 32 run down its rows
    const int64_t mem_rows = cols, mem_cols = rows;
    dim3 grid((unsigned)((mem_cols + kColsTC - 1) / kColsTC), (unsigned)((mem_rows + kColsTR - 1) / kColsTR));
    if (grid.y > 65535u) return km_fail(KM_ERR_ARG, "km_quant_mx: tensor too large for the transposing kernel");
    KM_DISPATCH_DT(dtype, hipLaunchKernelGGL((quant_cols<DT, true>), grid, dim3(kColsThreads), 0, st, xp, stride_col,
                                             mem_rows, mem_cols, qp, sp, kp, (const uint32_t*)nullptr));
  } else {
    const int64_t nb = rows * (cols / 32);
    KM_DISPATCH_DT(dtype, hipLaunchKernelGGL(quant_mx_generic<DT>, dim3((unsigned)((nb + 255) / 256)), dim3(256), 0, st,
                                             xp, stride_row, stride_col, rows, cols, qp, sp, kp));
  }
  return km_check_launch("km_quant_mx");
}

extern "C" int64_t km_scales_packed_bytes(int64_t rows, int64_t cols) {
  if (rows < 0 || cols < 0 || cols % 128) return -1;
  return (cols / 128) * ((rows + 127) / 128) * 512;
}

extern "C" int km_scales_pack(const void* scales, int64_t rows, int64_t cols, void* out, void* stream) {
  if (rows < 0 || cols < 0 || cols % 128) return km_fail(KM_ERR_ARG, "km_scales_pack: cols must be a multiple of 128");
  if (rows == 0 || cols == 0) return KM_OK;
  if (!scales || !out) return km_fail(KM_ERR_ARG, "km_scales_pack: null pointer");
  const int64_t n = rows * (cols / 32);
  hipLaunchKernelGGL(scales_pack, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (const uint8_t*)scales, rows, cols / 32, (uint8_t*)out);
  return km_check_launch("km_scales_pack");
}

extern "C" int km_quant_tensor(const void* x, int64_t rows, int64_t cols, int64_t stride_row,
                               int64_t stride_col, int dtype, void* q, float* scale_out,
                               uint32_t* amax_workspace, void* stream) {
  if (dtype != KM_BF16 && dtype != KM_F16) return km_fail(KM_ERR_ARG, "km_quant_tensor: dtype must be bf16 or f16");
  if (rows < 0 || cols < 0) return km_fail(KM_ERR_ARG, "km_quant_tensor: negative shape");
  if (!scale_out || !amax_workspace) return km_fail(KM_ERR_ARG, "km_quant_tensor: null scale or workspace");
  hipStream_t st = (hipStream_t)stream;
  const int64_t n = rows * cols;
  if (n > 0 && (!x || !q)) return km_fail(KM_ERR_ARG, "km_quant_tensor: null pointer");
  int64_t want = (n / 8 + 1023) / 1024;  // one 16 KiB piece per work-group and trip
  unsigned blocks = (unsigned)(want < 1 ? 1 : (want > kTensorBlocks ? kTensorBlocks : want));
  const int64_t amax_want = (n / 8 + kAmaxPiece - 1) / kAmaxPiece;
  const unsigned amax_blocks = (unsigned)(amax_want < 1 ? 1 : (amax_want > kAmaxBlocks ? kAmaxBlocks : amax_want));
  const uint16_t* xp = (const uint16_t*)x;
  KM_DISPATCH_DT(dtype, {
    if (n > 0) hipLaunchKernelGGL(tensor_amax<DT>, dim3(amax_blocks), dim3(kAmaxThreads), 0, st, xp, stride_row, stride_col, rows, cols, amax_workspace);
    hipLaunchKernelGGL(tensor_cast<DT>, dim3(blocks), dim3(256), 0, st, xp, stride_row, stride_col, rows, cols, amax_workspace, n > 0 ? (int)amax_blocks : 0, (uint8_t*)q, scale_out);
  });
  return km_check_launch("km_quant_tensor");
}

extern "C" int km_quant_rows(const void* x, int64_t rows, int64_t cols, int64_t stride_row, int64_t stride_col,
                             int dtype, void* q, float* scale_out, void* stream) {
  if (dtype != KM_BF16 && dtype != KM_F16) return km_fail(KM_ERR_ARG, "km_quant_rows: dtype must be bf16 or f16");
  if (rows < 0 || cols < 0) return km_fail(KM_ERR_ARG, "km_quant_rows: negative shape");
  if (rows == 0) return KM_OK;
  if (rows > 0x7FFFFFFFll) return km_fail(KM_ERR_ARG, "km_quant_rows: too many rows");
  if (!scale_out || (cols > 0 && (!x || !q))) return km_fail(KM_ERR_ARG, "km_quant_rows: null pointer");
  hipStream_t st = (hipStream_t)stream;
  const uint16_t* xp = (const uint16_t*)x;
  const dim3 grid((unsigned)((rows + 3) / 4));
  const bool aligned = (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(q) & 7) == 0;
  if (stride_col == 1 && aligned && cols % 8 == 0 && stride_row % 8 == 0 && stride_row >= cols && cols / 8 <= 0x7FFFFFFFll) {
    const uint32_t chunks = (uint32_t)(cols / 8);
    KM_DISPATCH_DT(dtype, {
      if (chunks <= 64u * kRowRecipeHeld)
        hipLaunchKernelGGL((quant_fp8_rows<DT, true>), grid, dim3(256), 0, st, xp, stride_row, chunks, (uint32_t)rows, (uint8_t*)q, scale_out);
      else
        hipLaunchKernelGGL((quant_fp8_rows<DT, false>), grid, dim3(256), 0, st, xp, stride_row, chunks, (uint32_t)rows, (uint8_t*)q, scale_out);
    });
  } else if (stride_row == 1 && aligned && (reinterpret_cast<uintptr_t>(q) & 15) == 0 && stride_col % 8 == 0 && stride_col >= rows &&
             rows % 8 == 0 && cols % 16 == 0 && (cols + kColsTR - 1) / kColsTR <= 65535) {
    // the memory is a row-major [cols][rows] matrix and q its transpose: column abs-max into
    // scale_out (as fp32 bits), transposing conversion, then the bits become the scales
    const int64_t mem_rows = cols, mem_cols = rows;
    uint32_t* bits = reinterpret_cast<uint32_t*>(scale_out);
    const dim3 tiles((unsigned)((mem_cols + kColsTC - 1) / kColsTC), (unsigned)((mem_rows + kColsTR - 1) / kColsTR));
    const dim3 amax_tiles((unsigned)((mem_cols + kAmaxTC - 1) / kAmaxTC), (unsigned)((mem_rows + kAmaxTR - 1) / kAmaxTR));
    const dim3 flat((unsigned)((rows + 255) / 256));
    hipLaunchKernelGGL(fill_u32_n, flat, dim3(256), 0, st, bits, rows, 0u);
    KM_DISPATCH_DT(dtype, {
      hipLaunchKernelGGL(cols_amax<DT>, amax_tiles, dim3(kColsThreads), 0, st, xp, stride_col, mem_rows, mem_cols, bits);
      hipLaunchKernelGGL((quant_cols<DT, false>), tiles, dim3(kColsThreads), 0, st, xp, stride_col, mem_rows, mem_cols,
                         (uint8_t*)q, (uint8_t*)nullptr, (uint8_t*)nullptr, (const uint32_t*)bits);
    });
    hipLaunchKernelGGL(amax_bits_to_scales, flat, dim3(256), 0, st, bits, rows);
  } else {
    KM_DISPATCH_DT(dtype, hipLaunchKernelGGL(quant_fp8_rows_generic<DT>, grid, dim3(256), 0, st, xp, stride_row, stride_col,
                                             (uint32_t)rows, cols, (uint8_t*)q, scale_out));
  }
  return km_check_launch("km_quant_rows");
}

extern "C" int km_quant_blocks(const void* x, int64_t rows, int64_t cols, int64_t stride_row, int64_t stride_col,
                               int dtype, int role, void* q, float* scale_out, float* scale_kmajor, void* stream) {
  if (dtype != KM_BF16 && dtype != KM_F16) return km_fail(KM_ERR_ARG, "km_quant_blocks: dtype must be bf16 or f16");
  if (role != KM_ROLE_ACT && role != KM_ROLE_WEIGHT) return km_fail(KM_ERR_ARG, "km_quant_blocks: role must be KM_ROLE_ACT or KM_ROLE_WEIGHT");
  if (rows < 0 || cols < 0 || cols % 128) return km_fail(KM_ERR_ARG, "km_quant_blocks: cols must be a non-negative multiple of 128");
  if (rows == 0 || cols == 0) return KM_OK;
  if (!x || !q || (!scale_out && !scale_kmajor)) return km_fail(KM_ERR_ARG, "km_quant_blocks: null pointer");
  if (role == KM_ROLE_WEIGHT && (scale_kmajor || !scale_out)) return km_fail(KM_ERR_ARG, "km_quant_blocks: weight blocks have the one scale layout");
  if (rows > 0x7FFFFFFFll) return km_fail(KM_ERR_ARG, "km_quant_blocks: too many rows");
  const int64_t tiles_x = cols / 128, tiles_y = (rows + 127) / 128;
  if (tiles_y > 65535 || tiles_x > 0x7FFFFFFFll) return km_fail(KM_ERR_ARG, "km_quant_blocks: tensor too large");
  hipStream_t st = (hipStream_t)stream;
  const uint16_t* xp = (const uint16_t*)x;
  const dim3 tiles((unsigned)tiles_x, (unsigned)tiles_y);
  const bool vec = stride_col == 1 && stride_row % 8 == 0 && stride_row >= cols && (reinterpret_cast<uintptr_t>(x) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(q) & 7) == 0;
  if (vec && role == KM_ROLE_ACT) {
    const uint64_t ngroups = (uint64_t)rows * (uint64_t)cols / 8;
    const uint64_t per_block = (uint64_t)kRowsThreads * kRowsUnroll;
    const uint64_t blocks = (ngroups + per_block - 1) / per_block;
    if (blocks > 0x7FFFFFFFull) return km_fail(KM_ERR_ARG, "km_quant_blocks: tensor too large");
    KM_DISPATCH_DT(dtype, hipLaunchKernelGGL(quant_fp8_blocks_act<DT>, dim3((unsigned)blocks), dim3(kRowsThreads), 0, st, xp, stride_row,
                                             (uint32_t)(cols / 8), ngroups, (uint32_t)rows, (uint8_t*)q, scale_out, scale_kmajor));
  } else if (vec) {
    KM_DISPATCH_DT(dtype, hipLaunchKernelGGL(quant_fp8_blocks_weight<DT>, tiles, dim3(256), 0, st, xp, stride_row, rows, cols, (uint8_t*)q, scale_out));
  } else if (role == KM_ROLE_ACT) {
    KM_DISPATCH_DT(dtype, hipLaunchKernelGGL((quant_fp8_blocks_generic<DT, false>), tiles, dim3(256), 0, st, xp, stride_row, stride_col, rows, cols, (uint8_t*)q, scale_out, scale_kmajor));
  } else {
    KM_DISPATCH_DT(dtype, hipLaunchKernelGGL((quant_fp8_blocks_generic<DT, true>), tiles, dim3(256), 0, st, xp, stride_row, stride_col, rows, cols, (uint8_t*)q, scale_out, (float*)nullptr));
  }
  return km_check_launch("km_quant_blocks");
}

extern "C" int km_quant_rows_i8(const void* x, int64_t rows, int64_t cols, int64_t stride_row, int64_t stride_col,
                                int dtype, const float* col_scale, void* q, float* scale_out, void* stream) {
  if (dtype != KM_BF16 && dtype != KM_F16) return km_fail(KM_ERR_ARG, "km_quant_rows_i8: dtype must be bf16 or f16");
  if (rows < 0 || cols < 0) return km_fail(KM_ERR_ARG, "km_quant_rows_i8: negative shape");
  if (rows == 0) return KM_OK;
  if (rows > 0x7FFFFFFFll) return km_fail(KM_ERR_ARG, "km_quant_rows_i8: too many rows");
  if (!scale_out || (cols > 0 && (!x || !q))) return km_fail(KM_ERR_ARG, "km_quant_rows_i8: null pointer");
  hipStream_t st = (hipStream_t)stream;
  const uint16_t* xp = (const uint16_t*)x;
  const dim3 grid((unsigned)((rows + 3) / 4));
  const bool aligned = (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(q) & 7) == 0 &&
                       (reinterpret_cast<uintptr_t>(col_scale) & 15) == 0;
  if (stride_col == 1 && aligned && cols % 8 == 0 && stride_row % 8 == 0 && stride_row >= cols && cols / 8 <= 0x7FFFFFFFll) {
    const uint32_t chunks = (uint32_t)(cols / 8);
    KM_DISPATCH_DT(dtype, {
      if (chunks <= 64u * kRowRecipeHeld)
        hipLaunchKernelGGL((quant_i8_rows<DT, true>), grid, dim3(256), 0, st, xp, stride_row, chunks, (uint32_t)rows, col_scale, (uint8_t*)q, scale_out);
      else
        hipLaunchKernelGGL((quant_i8_rows<DT, false>), grid, dim3(256), 0, st, xp, stride_row, chunks, (uint32_t)rows, col_scale, (uint8_t*)q, scale_out);
    });
  } else {
    KM_DISPATCH_DT(dtype, hipLaunchKernelGGL(quant_i8_rows_generic<DT>, grid, dim3(256), 0, st, xp, stride_row, stride_col,
                                             (uint32_t)rows, cols, col_scale, (uint8_t*)q, scale_out));
  }
  return km_check_launch("km_quant_rows_i8");
}

extern "C" int km_quant_rows_i8_rotated(const void* x, int64_t rows, int64_t cols, int64_t stride_row, int dtype, int group,
                                        void* q, float* scale_out, void* stream) {
  if (dtype != KM_BF16 && dtype != KM_F16) return km_fail(KM_ERR_ARG, "km_quant_rows_i8_rotated: dtype must be bf16 or f16");
  int stages = 0;
  for (int g = group; g > 1 && g % 4 == 0; g /= 4) ++stages;
  if (group < 4 || (1 << (2 * stages)) != group || stages > 5)
    return km_fail(KM_ERR_ARG, "km_quant_rows_i8_rotated: group must be 4, 16, 64, 256 or 1024");
  if (rows < 0 || cols < 0 || cols % group) return km_fail(KM_ERR_ARG, "km_quant_rows_i8_rotated: cols must be a non-negative multiple of the group");
  if (rows == 0 || cols == 0) return KM_OK;
  if (rows > 0x7FFFFFFFll) return km_fail(KM_ERR_ARG, "km_quant_rows_i8_rotated: too many rows");
  if (!x || !q || !scale_out) return km_fail(KM_ERR_ARG, "km_quant_rows_i8_rotated: null pointer");
  if (group < 16 || cols > kRotMaxCols || stride_row % 8 || stride_row < cols || (reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(q) & 15))
    return km_fail(KM_ERR_UNSUPPORTED, "km_quant_rows_i8_rotated: groups of 16 and more, rows of up to 4096 elements, 16-byte aligned operands, row stride a multiple of 8");
  hipStream_t st = (hipStream_t)stream;
  const uint16_t* xp = (const uint16_t*)x;
  const dim3 grid((unsigned)rows);
#define KM_ROT_CASE(J) hipLaunchKernelGGL((rotate_quant_i8_rows<DT, J>), grid, dim3(256), 0, st, xp, stride_row, (uint32_t)cols, (uint8_t*)q, scale_out)
  KM_DISPATCH_DT(dtype, {
    switch (stages) {
      case 2: KM_ROT_CASE(2); break;
      case 3: KM_ROT_CASE(3); break;
      case 4: KM_ROT_CASE(4); break;
      default: KM_ROT_CASE(5); break;
    }
  });
#undef KM_ROT_CASE
  return km_check_launch("km_quant_rows_i8_rotated");
}
