// The weight-only dequant-GEMM kernel template and its launchers, shared by the translation units
// of the forward (km_wo_gemm.hip) and of the input gradient over the stored codes (km_wo_dgrad.hip).
#pragma once
#include <hip/hip_fp16.h>
#include <stdio.h>

#include "km_gemm_common.h"
#include "km_wo_tiles.h"

namespace km {

constexpr int kWoStepElems = 64;  // contraction elements per step (128 B of 16-bit values)

template <int DT>
__device__ __forceinline__ void mfma16(v4f& c, const v4i& a, const v4i& b) {
  if constexpr (DT == KM_BF16)
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  else
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}

typedef float v2f __attribute__((ext_vector_type(2)));

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

// 8 codes (two dwords) -> 8 values of the activation type (four dwords); `s` scales them in
// fp32 before the single rounding (dgrad), or is unused (forward: the conversion is exact)
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

// d[i] holds the codes (n = i, k = 0..3) of eight rows; o[j] gets the codes (k = j, n = 0..7).
// __builtin_amdgcn_perm(hi, lo, sel): byte i of the result is byte sel[i] of {lo: 0-3, hi: 4-7}.
__device__ __forceinline__ void transpose_8x4(const uint32_t (&d)[8], uint2 (&o)[4]) {
  uint32_t half[2][4];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const uint32_t* r = d + 4 * h;
    const uint32_t a01 = __builtin_amdgcn_perm(r[1], r[0], 0x05010400u), b01 = __builtin_amdgcn_perm(r[1], r[0], 0x07030602u);
    const uint32_t a23 = __builtin_amdgcn_perm(r[3], r[2], 0x05010400u), b23 = __builtin_amdgcn_perm(r[3], r[2], 0x07030602u);
    half[h][0] = __builtin_amdgcn_perm(a23, a01, 0x05040100u);
    half[h][1] = __builtin_amdgcn_perm(a23, a01, 0x07060302u);
    half[h][2] = __builtin_amdgcn_perm(b23, b01, 0x05040100u);
    half[h][3] = __builtin_amdgcn_perm(b23, b01, 0x07060302u);
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) o[j] = make_uint2(half[0][j], half[1][j]);
}

// Epilogue of the input-gradient kernel that reads q as stored. Row 16 t + r of a wavefront's B
// slab holds column 64 b + 4 r + j of the wavefront's WTN columns, t = j Q + b, Q = WTN / 64: lane
// (r16, g) holds, for every b, the sixteen consecutive columns 64 b + 16 g .. + 15 of output row
// r16, element v of tile j Q + b being column 64 b + 16 g + 4 v + j. A 96-column wavefront has
// tiles 0-3 laid out like that (b = 0) and its columns 64 .. 95 in tiles 4 and 5: row i of tile 4
// is column 64 + 4 (i % 8) + i / 8, of tile 5 column 64 + 4 (i % 8) + 2 + i / 8, so the lower 32
// lanes hold residues 0 and 2 of columns 64 + 16 g + 4 v .. + 3 and the lanes 32 places up
// residues 1 and 3: V_PERMLANE32_SWAP brings them together and the lower lanes write the piece.
// Interior tiles go through the same LDS staging as store_tile (8-byte LDS writes, 16-byte reads
// along rows, full-line global stores); edge tiles store four columns at a time (NO % 4 == 0
// here). No scale, no bias.
template <int BM, int BN, int OUT>
__device__ __forceinline__ void store_tile_by_fours(v4f (&acc)[BN / 32][BM / 32], uint16_t* __restrict__ C, int M, int NO, int m0,
                                                    int n0, uint8_t* buf0, uint8_t* buf1, uint8_t* buf2, uint8_t* buf3) {
  constexpr int WTM = BM / 2, WTN = BN / 2, TM = WTM / 16, Q = WTN / 64;
  constexpr bool kTail = WTN % 64 != 0;  // 32 more columns in the last two tiles
  static_assert(BN / 32 == 4 * Q + (kTail ? 2 : 0) && (!kTail || WTN % 64 == 32), "four column residues per 64 columns");
  const int tid = fresh_thread_index();  // see store_tile
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6) & 3;
  const int wm = (wave >> 1) * WTM, wn = (wave & 1) * WTN;
  const int r16 = lane & 15, g = lane >> 4;
  // every accumulator element is read by an opaque statement at its use (see store_tile)
  auto four = [&](int b, int j, int v) __attribute__((always_inline)) {
    return make_uint2(pack2<OUT>(acc_element<true>(acc[b][j], v), acc_element<true>(acc[Q + b][j], v)),
                      pack2<OUT>(acc_element<true>(acc[2 * Q + b][j], v), acc_element<true>(acc[3 * Q + b][j], v)));
  };
  // the piece of the tail tiles: valid in the lower 32 lanes (g < 2), columns 64 Q + 16 g + 4 v .. + 3
  auto tail_four = [&](int j, int v) __attribute__((always_inline)) {
    const uint32_t x = __builtin_bit_cast(uint32_t, acc_element<true>(acc[4 * Q][j], v));
    const uint32_t y = __builtin_bit_cast(uint32_t, acc_element<true>(acc[4 * Q + 1][j], v));
    const auto xs = __builtin_amdgcn_permlane32_swap(x, x, false, false);  // [1]: the value 32 lanes up
    const auto ys = __builtin_amdgcn_permlane32_swap(y, y, false, false);
    return make_uint2(pack2<OUT>(__builtin_bit_cast(float, x), __builtin_bit_cast(float, (uint32_t)xs[1])),
                      pack2<OUT>(__builtin_bit_cast(float, y), __builtin_bit_cast(float, (uint32_t)ys[1])));
  };
  if (m0 + BM <= M && n0 + BN <= NO && (NO & 7) == 0) {
    __syncthreads();  // every wavefront is done reading fragments
    uint8_t* region = wave == 0 ? buf0 : wave == 1 ? buf1 : wave == 2 ? buf2 : buf3;
    uint8_t* out_base = reinterpret_cast<uint8_t*>(C) + ((size_t)(m0 + wm) * NO + n0 + wn) * 2;
    // piece t = 4 b + v of a pass: the columns 64 b + 16 g + 4 v .. + 3 of this lane's row; the
    // four pieces after those are the tail's (no write from the upper lanes: offset -1)
    staged_rows_out<WTN, TM, 4 * Q + (kTail ? 4 : 0)>(
        region, out_base, NO, lane,
        [&](auto j_tag, auto t_tag) __attribute__((always_inline)) {
          constexpr int j = decltype(j_tag)::value, t = decltype(t_tag)::value;
          if constexpr (t < 4 * Q) return four(t / 4, j, t % 4);
          else return tail_four(j, t - 4 * Q);
        },
        [&](int t) __attribute__((always_inline)) { return t < 4 * Q ? (64 * (t / 4) + 16 * g + 4 * (t % 4)) * 2 : g < 2 ? (64 * Q + 16 * g + 4 * (t - 4 * Q)) * 2 : -1; });
    return;
  }
#pragma unroll
  for (int j = 0; j < TM; ++j) {
    const int m = m0 + wm + j * 16 + r16;
#pragma unroll
    for (int b = 0; b < Q; ++b)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int col = n0 + wn + 64 * b + 16 * g + 4 * v;
        const uint2 piece = four(b, j, v);
        if (m < M && col < NO) *reinterpret_cast<uint2*>(C + (size_t)m * NO + col) = piece;
      }
    if constexpr (kTail) {
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int col = n0 + wn + 64 * Q + 16 * g + 4 * v;
        const uint2 piece = tail_four(j, v);  // every lane takes part in the exchange
        if (g < 2 && m < M && col < NO) *reinterpret_cast<uint2*>(C + (size_t)m * NO + col) = piece;
      }
    }
  }
}

// two codes (byte pair `pair` of word w) -> one dword of two values of the activation type, each
// scaled in fp32 before its single rounding when SCALE is set
template <int DT, int QF, bool SCALE>
__device__ __forceinline__ uint32_t widen_pair(uint32_t w, int pair, float s0, float s1) {
  if constexpr (QF == KM_Q_E4M3 && !SCALE) {
    if constexpr (DT == KM_BF16)
      return pair ? __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true))
                  : __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false));
    else
      return pair ? __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, true))
                  : __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, false));
  } else {
    float f0, f1;
    if constexpr (QF == KM_Q_E4M3) {
      const v2f v = pair ? __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true) : __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
      f0 = v.x;
      f1 = v.y;
    } else {
      f0 = (float)(int)(int8_t)((w >> (16 * pair)) & 0xFFu);
      f1 = (float)(int)(int8_t)((w >> (16 * pair + 8)) & 0xFFu);
    }
    if constexpr (SCALE) {
      f0 *= s0;
      f1 *= s1;
    }
    return pack2<DT>(f0, f1);
  }
}

// Half of an 8 x 4 byte transposition is all the widening needs: a dword of two values holds one
// column of rows 2d, 2d+1, and a byte permute of two row dwords gives two such pairs. p = 4 h + i:
// rows 4h .. 4h+3 of d, i = 0: columns 0,1 of rows 0,1 (bytes r0c0 r1c0 r0c1 r1c1); 1: columns 2,3 of
// rows 0,1; 2, 3: the same of rows 2,3.
__device__ __forceinline__ uint32_t pair_rows(const uint32_t (&d)[8], int p) {
  const uint32_t* r = d + 4 * (p >> 2) + 2 * ((p >> 1) & 1);
  return __builtin_amdgcn_perm(r[1], r[0], (p & 1) ? 0x07030602u : 0x05010400u);
}

// how the codes are laid out and scaled
enum { kWoFwd = 0, kWoDgradT = 1, kWoDgradN = 2 };
// kWoFwd     codes [NO, KC]; scale fp32 [NO] applied with the bias in the epilogue
// kWoDgradT  codes [NO, KC] (a transposed copy of q); scale fp32 [KC] applied before the rounding
// kWoDgradN  codes [KC, NO] (q as stored); scale(n, k) by SK, applied before the rounding

// LDS layout of a 32-deep slab: a row is 64 bytes (four 16-byte chunks of eight 16-bit values),
// rows in order, sixteen rows fill 1 KiB; the chunk index is XORed with (row / 2) % 4. A 16-byte
// LDS access is served eight lanes at a time, 128 bytes a cycle: eight consecutive lanes must hit
// eight different 16-byte slots modulo 128 bytes. Eight lanes that read one chunk of eight
// consecutive rows (an MFMA fragment read, or the transposing mode's writes) do: two rows share a
// 128-byte line and the four lines differ in the XOR key; so do eight lanes that write the four
// chunks of two consecutive rows. (A layout that spread 16 lanes over 256 bytes instead measured
// bank conflicts in 40-50 % of the LDS-active cycles.)
__device__ __forceinline__ int slab32_offset(int row, int chunk) {
  return (row << 6) + ((chunk ^ ((row >> 1) & 3)) << 4);
}

// In-loop forms without the wait states for a vector-ALU-written SGPR: inside the K loop every SGPR
// these read is loop invariant or written by the scalar ALU (m0 still needs its one wait state).
__device__ __forceinline__ uint64_t loop_load_b64(const v4i& rsrc, int voffset) {
  uint64_t v;
  asm volatile("buffer_load_dwordx2 %0, %1, %2, 0 offen" : "=v"(v) : "v"(voffset), "s"(rsrc) : "memory");
  return v;
}
__device__ __forceinline__ uint32_t loop_load_b32(const v4i& rsrc, int voffset) {
  uint32_t v;
  asm volatile("buffer_load_dword %0, %1, %2, 0 offen" : "=v"(v) : "v"(voffset), "s"(rsrc) : "memory");
  return v;
}
typedef uint64_t v4u64 __attribute__((ext_vector_type(4)));
// scalar load of eight dwords (as four pairs) at a wavefront-uniform byte offset; past the descriptor's size reads as zero
__device__ __forceinline__ v4u64 loop_sload_x8(const v4i& rsrc, int soffset) {
  v4u64 v;
  asm volatile("s_buffer_load_dwordx8 %0, %1, %2" : "=s"(v) : "s"(rsrc), "s"(soffset) : "memory");
  return v;
}
__device__ __forceinline__ v4i loop_load_b128(const v4i& rsrc, int voffset) {
  v4i v;
  asm volatile("buffer_load_dwordx4 %0, %1, %2, 0 offen" : "=v"(v) : "v"(voffset), "s"(rsrc) : "memory");
  return v;
}
__device__ __forceinline__ uint32_t loop_load_u8(const v4i& rsrc, int voffset) {
  uint32_t v;
  asm volatile("buffer_load_ubyte %0, %1, %2, 0 offen" : "=v"(v) : "v"(voffset), "s"(rsrc) : "memory");
  return v;
}
__device__ __forceinline__ uint32_t hidden_load_u8(const v4i& rsrc, int voffset) {
  uint32_t v;
  asm volatile("s_nop 4\n\tbuffer_load_ubyte %0, %1, %2, 0 offen" : "=v"(v) : "v"(voffset), "s"(rsrc) : "memory");
  return v;
}

template <int BM, int BN, int DT, int QF, int MODE, int SK>
__global__ __launch_bounds__(256) void wo_gemm_kernel(const uint16_t* __restrict__ A, const uint8_t* __restrict__ Q,
                                                      const void* __restrict__ scale_ptr, int scale_ld,
                                                      const uint16_t* __restrict__ bias, uint16_t* __restrict__ C, int M, int NO,
                                                      int KC, int tn_first, int tn_count) {
  // the grid covers tile columns tn_first .. tn_first + tn_count - 1 of the output
  constexpr int WTM = BM / 2, WTN = BN / 2;
  constexpr int TM = WTM / 16, TN = WTN / 16;
  constexpr int STAGES = 4;
  constexpr int A_STAGE = BM * 64, B_STAGE = BN * 64;  // bytes of one 32-deep slab
  constexpr int A_LD = BM / 64;                        // direct-to-LDS passes per step: 16 rows per wavefront and pass
  constexpr bool NAT = MODE == kWoDgradN;
  constexpr bool PRESCALE = MODE != kWoFwd;
  constexpr int UNITS = NAT ? 4 : BN / 64;             // 16-byte LDS writes per thread and step
  // Codes as stored, 128 columns: the 32 dwords of a row n keep half a wavefront busy, so the
  // halves take four rows n each (everything per lane and step halves: loads, permutes,
  // conversions, scale bytes; a lane writes 8 bytes per column instead of 16).
  constexpr bool kHalfRows = NAT && BN == 128;
  constexpr bool kHalfRowScales = kHalfRows && SK == KM_WSCALE_ROWS;  // four fp32 row scales in one vector load
  constexpr int NROWS = kHalfRows ? 4 : 8;             // rows n per lane (codes as stored)
  constexpr int DPC = NROWS / 2;                       // dwords of two values per column
  constexpr int NQ = NAT ? NROWS : UNITS;              // code loads per thread and step
  constexpr int NS = !NAT ? 0 : SK == KM_WSCALE_E8M0 ? NROWS : (SK == KM_WSCALE_BLOCKS || kHalfRowScales) ? 1 : 0;  // scale loads through the vector path
  constexpr int NV = A_LD + NQ + NS;                   // vector-memory loads issued per step, counted by hand below
  static_assert(!NAT || BN == 256 || BN == 192 || BN == 128, "the transposing load covers 256, 192 or 128 columns");
  static_assert(NV < 48, "vmcnt holds 6 bits");
  __shared__ __attribute__((aligned(1024))) uint8_t a_ring[STAGES * A_STAGE];
  __shared__ __attribute__((aligned(1024))) uint8_t b_ring[STAGES * B_STAGE];

  int tile_m, tile_n;
  tile_of(blockIdx.x, (M + BM - 1) / BM, tn_count, tile_m, tile_n, kGroupMWideA);
  const int m0 = tile_m * BM, n0 = (tn_first + tile_n) * BN;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = (wave >> 1) * WTM, wn = (wave & 1) * WTN;
  const int r16 = lane & 15, g = lane >> 4;
  // steps of 32 contraction elements, in rounds of four (the ring's stages and the two register
  // sets are compile-time positions of a round): a padded step multiplies slabs of zeros
  const int steps = ((KC + 31) / 32 + 3) & ~3;
  constexpr int kOob = 0x7FFFFFFF;  // an offset past every buffer: the load returns 0

  const v4i a_rsrc = raw_rsrc(A + (size_t)m0 * KC, (uint32_t)min((int64_t)(M - m0) * KC * 2, (int64_t)0x7FFFFFFF));
  // K-contiguous codes: the tile's rows start at n0; codes as stored: its columns start at n0
  const int64_t q_skip = NAT ? (int64_t)n0 : (int64_t)n0 * KC;
  const v4i q_rsrc = raw_rsrc(Q + q_skip, (uint32_t)min((int64_t)NO * KC - q_skip, (int64_t)0x7FFFFFFF));

  // direct-to-LDS A pass: lane L lands in 16-byte slot L of its wavefront's 1 KiB block, which is
  // (row L / 4, chunk (L % 4) ^ (L / 8) % 4) of the block in the slab layout
  const int dma_row = wave * 16 + (lane >> 2);
  const int dma_chunk = (lane & 3) ^ ((lane >> 3) & 3);
  // K-contiguous codes: four lanes cover the 32 codes of a row, a wavefront 16 rows, a unit 64 rows
  const int q_row = wave * 16 + (lane >> 2), q_chunk = lane & 3;
  // codes as stored: LPR lanes cover the BN columns of one row n with a dword each (the other lanes
  // of a 128-column tile load nothing and write nothing); wavefront w owns rows n = 8 w .. 8 w + 7
  // of the step's 32, which become chunk w of the slab rows
  constexpr int LPR = BN / 4;
  const bool nat_live = kHalfRows || lane < LPR;
  const int row_half = kHalfRows ? lane / LPR : 0;           // rows n = 8 wave + 4 row_half .. + 3
  const int col4 = lane % LPR;                               // columns 4 col4 .. 4 col4 + 3 of the tile
  const int half_w = col4 / (LPR / 2), col_l = col4 % (LPR / 2);
  // slab row of column j: nat_row0 + j * nat_stride. A wavefront's WTN / 4 dwords per row n are laid
  // out so that every 16-row MFMA tile holds one j: with WTN / 4 a multiple of 16, j-major; with the
  // 24 dwords of a 96-column half, dwords 0-15 j-major in tiles 0-3 and dwords 16-23 as rows
  // 64 + 8 j + (dword - 16) of tiles 4 and 5 (see store_tile_by_fours)
  constexpr bool kNatWhole = (WTN / 4) % 16 == 0;
  const int nat_row0 = half_w * WTN + (kNatWhole || col_l < 16 ? col_l : 48 + col_l);
  const int nat_stride = kNatWhole ? WTN / 4 : col_l < 16 ? 16 : 8;

  const int a_frag = lds_offset(a_ring) + slab32_offset(wm + r16, g);  // + j KiB + stage
  const int b_frag = lds_offset(b_ring) + slab32_offset(wn + r16, g);  // + t KiB + stage

  v4f acc[TN][TM];

  // codes and scales in flight, set s & 1 for slab s
  uint32_t raw[2][NAT ? 8 : 2 * UNITS];
  float sc[2][8];
  uint32_t sraw[2][kHalfRows ? 4 : NS ? NS : 1];
#pragma unroll
  for (int b = 0; b < 2; ++b)
#pragma unroll
    for (int i = 0; i < 8; ++i) sc[b][i] = 1.f;

  // row scales of codes as stored: eight per slab and wavefront, wavefront-uniform
  constexpr bool kRowScalars = NAT && SK == KM_WSCALE_ROWS && !kHalfRows;
  v4u64 scr[2] = {};
  v4i row_scale_rsrc = v4i{0, 0, 0, 0};
  uint64_t tensor_scale_twice = 0;  // zero with row scales
  if constexpr (kRowScalars || kHalfRowScales) {
    row_scale_rsrc = raw_rsrc(scale_ptr, scale_ld ? (uint32_t)KC * 4u : 4u);
    const uint32_t bits = scale_ld ? 0u : (uint32_t)__builtin_amdgcn_readfirstlane(*static_cast<const int*>(scale_ptr));
    tensor_scale_twice = ((uint64_t)bits << 32) | bits;
  }
  v4i scale_rsrc = v4i{0, 0, 0, 0};
  if constexpr (NS > 0) {
    const int64_t bytes = SK == KM_WSCALE_E8M0 ? (int64_t)KC * scale_ld : (int64_t)((KC + 127) >> 7) * scale_ld * 4;
    scale_rsrc = raw_rsrc(scale_ptr, (uint32_t)min(bytes, (int64_t)0x7FFFFFFF));
  }

  auto opaque = [](int v) __attribute__((always_inline)) {
    asm volatile("" : "+v"(v));
    return v;
  };
  // Columns past KC become out-of-range offsets (whole 8-element chunks, KC % 8 == 0), rows past the
  // end are out of range by themselves: both read as zeros. One per-lane offset per slab, made
  // opaque so that the optimizer does not carry an induction register per pass; a pass adds a
  // uniform row stride (kOob plus a stride stays out of range: the hardware compares unsigned).
  auto a_offset = [&](int s) __attribute__((always_inline)) {
    const int col = s * 32 + dma_chunk * 8;
    return opaque(col < KC ? (dma_row * KC + col) * 2 : kOob);
  };
  auto dma_a_pass = [&](int stage, int a_off, int i) __attribute__((always_inline)) {
    loop_dma_b128(a_rsrc, lds_offset(a_ring) + stage * A_STAGE + (i * 4 + wave) * 1024, a_off + i * (64 * 2) * KC, 0);
  };
  // K-contiguous codes: one per-lane offset per slab, as for A
  auto q_offset = [&](int s) __attribute__((always_inline)) {
    if constexpr (NAT) return 0;
    else {
      const int col = s * 32 + q_chunk * 8;
      return opaque(col < KC ? q_row * KC + col : kOob);
    }
  };
  // Codes as stored: the descriptor of slab s starts at row 32 s of q and ends where q ends, so the
  // offsets of a lane's eight rows (n = 32 s + 8 wave + i, four columns) do not depend on s, rows
  // past the end stay out of range and the walk from slab to slab is scalar arithmetic.
  int q_voff[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) q_voff[i] = NAT && i < NROWS ? opaque(nat_live ? (8 * wave + 4 * row_half + i) * NO + 4 * col4 : kOob) : 0;
  const int q_slab_bytes = 32 * NO;
  const uint64_t q_first = (uint64_t)reinterpret_cast<uintptr_t>(Q) + (uint64_t)q_skip;
  int q_walk_lo = __builtin_amdgcn_readfirstlane((int)(uint32_t)q_first);
  int q_walk_hi = __builtin_amdgcn_readfirstlane((int)((uint32_t)(q_first >> 32) & 0xFFFFu));
  int q_walk_left = __builtin_amdgcn_readfirstlane((int)min((int64_t)NO * KC - q_skip, (int64_t)0x7FFFFFFF));
  auto q_walk_rsrc = [&]() __attribute__((always_inline)) { return v4i{q_walk_lo, q_walk_hi, max(q_walk_left, 0), 0x00020000}; };
  auto q_walk_advance = [&]() __attribute__((always_inline)) {
    // the bytes left go negative past the end (by at most 127 rows: no wrap) and are clamped above
    asm volatile("s_add_u32 %0, %0, %3\n\ts_addc_u32 %1, %1, 0\n\ts_sub_i32 %2, %2, %3"
                 : "+s"(q_walk_lo), "+s"(q_walk_hi), "+s"(q_walk_left) : "s"(q_slab_bytes) : "scc");
  };
  // piece i of the code loads of a slab into register set `set` (codes as stored: of the slab the
  // walking descriptor stands at)
  auto load_code_piece = [&](int set, int q_off, int i) __attribute__((always_inline)) {
    if constexpr (!NAT) {
      const uint64_t v = loop_load_b64(q_rsrc, q_off + i * 64 * KC);
      raw[set][2 * i] = (uint32_t)v;
      raw[set][2 * i + 1] = (uint32_t)(v >> 32);
    } else {
      raw[set][i] = loop_load_b32(q_walk_rsrc(), q_voff[i]);
    }
  };
  // Scales of slab s. Rows and columns past the end are clamped: their codes are zeros or belong
  // to outputs that are never stored, the scale only has to come from valid memory.
  auto scale_offset = [&](int s) __attribute__((always_inline)) {
    if constexpr (NS == 0) return 0;
    else if constexpr (kHalfRowScales) return opaque(min(s * 32 + 8 * wave + 4 * row_half, KC - 4) * 4);  // four row scales
    else {
      const int n = min(s * 32 + 8 * wave + 4 * row_half, KC - NROWS);
      const int k = min(n0 + 4 * col4, NO - 1);  // this thread's first output column (a column of q)
      if constexpr (SK == KM_WSCALE_E8M0) return opaque(n * scale_ld + (k >> 5));
      else return opaque(((n >> 7) * scale_ld + (k >> 7)) * 4);  // n .. n + 7 share a block
    }
  };
  auto load_scale_piece = [&](int set, int s_off, int i) __attribute__((always_inline)) {
    if constexpr (kHalfRowScales) {
      // range-checked: with one scale for the whole tensor every dword but the one at offset 0 reads as zero
      const v4i v = loop_load_b128(row_scale_rsrc, s_off);
      sraw[set][0] = (uint32_t)v[0]; sraw[set][1] = (uint32_t)v[1]; sraw[set][2] = (uint32_t)v[2]; sraw[set][3] = (uint32_t)v[3];
    } else if constexpr (SK == KM_WSCALE_E8M0) sraw[set][i] = loop_load_u8(scale_rsrc, s_off + i * scale_ld);
    else sraw[set][0] = loop_load_b32(scale_rsrc, s_off);
  };
  // scales that do not go through the counted vector loads: per contraction column of a transposed
  // copy (two 16-byte loads), per row of q as stored (wavefront-uniform: scalar loads)
  auto load_scalar_scales = [&](int set, int s) __attribute__((always_inline)) {
    if constexpr (MODE == kWoDgradT) {
      const float* scale = static_cast<const float*>(scale_ptr);
      const int col = min(s * 32 + q_chunk * 8, KC - 8);  // whole chunks: KC % 8 == 0
      const float4 lo = *reinterpret_cast<const float4*>(scale + col), hi = *reinterpret_cast<const float4*>(scale + col + 4);
      sc[set][0] = lo.x; sc[set][1] = lo.y; sc[set][2] = lo.z; sc[set][3] = lo.w;
      sc[set][4] = hi.x; sc[set][5] = hi.y; sc[set][6] = hi.z; sc[set][7] = hi.w;
    } else if constexpr (kRowScalars) {
      // eight consecutive scales in one range-checked scalar load (with one scale for the whole
      // tensor every offset but 0 is out of range and reads as zero)
      const int n = min(s * 32 + 8 * wave, KC - 8);  // wavefront-uniform
      scr[set] = loop_sload_x8(row_scale_rsrc, n * 4);
    }
  };
  // The scalar load is an opaque statement: its registers are read here, one step-end wait later.
  // Row scales pass through; of a per-tensor scale the load brought zeros (or the scale itself, at
  // offset 0), and the scale is ORed over every one, two at a time.
  auto merge_scales = [&](int set) __attribute__((always_inline)) {
    if constexpr (kRowScalars) {
      uint64_t r[4];
      asm volatile("s_or_b64 %0, %4, %8\n\ts_or_b64 %1, %5, %8\n\ts_or_b64 %2, %6, %8\n\ts_or_b64 %3, %7, %8"
                   : "=&s"(r[0]), "=&s"(r[1]), "=&s"(r[2]), "=&s"(r[3])
                   : "s"(scr[set][0]), "s"(scr[set][1]), "s"(scr[set][2]), "s"(scr[set][3]), "s"(tensor_scale_twice)
                   : "scc");
#pragma unroll
      for (int i = 0; i < 8; ++i) sc[set][i] = bits_f32((uint32_t)(r[i >> 1] >> (32 * (i & 1))));
    } else if constexpr (kHalfRowScales) {
#pragma unroll
      for (int i = 0; i < 4; ++i) sc[set][i] = bits_f32(sraw[set][i] | (uint32_t)tensor_scale_twice);
    }
  };
  auto load_slab = [&](int set, int s) __attribute__((always_inline)) {
    load_scalar_scales(set, s);
    const int q_off = q_offset(s), s_off = scale_offset(s);
#pragma unroll
    for (int i = 0; i < NS; ++i) load_scale_piece(set, s_off, i);
#pragma unroll
    for (int i = 0; i < NQ; ++i) load_code_piece(set, q_off, i);
    if constexpr (NAT) q_walk_advance();  // slabs are requested in order: 0 .. 3 here, s + 4 in step s
  };
  auto dma_a = [&](int stage, int s) __attribute__((always_inline)) {
    const int a_off = a_offset(s);
#pragma unroll
    for (int i = 0; i < A_LD; ++i) dma_a_pass(stage, a_off, i);
  };
  // The widen-and-store work of a slab in single-instruction pieces, so that each can ride behind
  // one MFMA. Codes as stored: eight byte permutes turn the eight dwords (n, 4 k) into words of two
  // byte pairs (k, rows 2d and 2d+1) `t1`. Then dword d of unit c (two values of the activation
  // type) comes from one byte pair, and unit c (four dwords) is one 16-byte LDS write.
  uint32_t t1[8], w16[UNITS][4];
  auto transpose_piece = [&](int set, int p) __attribute__((always_inline)) {  // p < NROWS
    if constexpr (NAT && QF != KM_Q_INT8) t1[p] = pair_rows(raw[set], p);  // an int8 conversion selects its byte by itself
  };
  auto widen_piece = [&](int set, int c, int d) __attribute__((always_inline)) {
    if constexpr (!NAT) {
      w16[c][d] = widen_pair<DT, QF, PRESCALE>(raw[set][2 * c + (d >> 1)], d & 1, sc[set][2 * d], sc[set][2 * d + 1]);
    } else {
      float s0, s1;
      if constexpr (SK == KM_WSCALE_ROWS) { s0 = sc[set][2 * d]; s1 = sc[set][2 * d + 1]; }
      else if constexpr (SK == KM_WSCALE_E8M0) { s0 = bits_f32(sraw[set][2 * d] << 23); s1 = bits_f32(sraw[set][2 * d + 1] << 23); }
      else { s0 = s1 = bits_f32(sraw[set][0]); }
      if constexpr (QF == KM_Q_INT8) {
        const float f0 = (float)(int)(int8_t)((raw[set][2 * d] >> (8 * c)) & 0xFFu) * s0;
        const float f1 = (float)(int)(int8_t)((raw[set][2 * d + 1] >> (8 * c)) & 0xFFu) * s1;
        w16[c][d] = pack2<DT>(f0, f1);
      } else {
        w16[c][d] = widen_pair<DT, QF, true>(t1[2 * d + (c >> 1)], c & 1, s0, s1);  // column c, rows 2d, 2d+1
      }
    }
  };
  auto store_unit = [&](int stage, int c) __attribute__((always_inline)) {
    uint8_t* slab = b_ring + stage * B_STAGE;
    if constexpr (kHalfRows) {
      *reinterpret_cast<uint2*>(slab + slab32_offset(nat_row0 + c * nat_stride, wave) + 8 * row_half) = make_uint2(w16[c][0], w16[c][1]);
    } else {
      const uint4 v = make_uint4(w16[c][0], w16[c][1], w16[c][2], w16[c][3]);
      if constexpr (!NAT) *reinterpret_cast<uint4*>(slab + slab32_offset(q_row + c * 64, q_chunk)) = v;
      else if (nat_live) *reinterpret_cast<uint4*>(slab + slab32_offset(nat_row0 + c * nat_stride, wave)) = v;
    }
  };
  auto commit_all = [&](int set, int stage) __attribute__((always_inline)) {
    merge_scales(set);
#pragma unroll
    for (int p = 0; p < NROWS; ++p) transpose_piece(set, p);
#pragma unroll
    for (int c = 0; c < UNITS; ++c) {
#pragma unroll
      for (int d = 0; d < (NAT ? DPC : 4); ++d) widen_piece(set, c, d);
      store_unit(stage, c);
    }
  };

  // MFMA operands of the current step and of the next, set s & 1 for step s
  v4i xf[2][TM], wf[2][TN];
  typedef __attribute__((address_space(3))) const v4i* lds_v4i_cptr;
  auto read_fragment = [&](int set, int stage, int r) __attribute__((always_inline)) {
    // r < TM: A fragment r; else B fragment r - TM
    if (r < TM) xf[set][r] = *(lds_v4i_cptr)(uint32_t)(a_frag + stage * A_STAGE + r * 1024);
    else wf[set][r - TM] = *(lds_v4i_cptr)(uint32_t)(b_frag + stage * B_STAGE + (r - TM) * 1024);
  };

  // Step s (position u = s % 4 of its round) multiplies slab s out of registers that were filled
  // during step s-1, and behind its MFMAs
  //   starts the A loads of slab s+3 (direct to LDS, stage (u+3) % 4),
  //   reads the fragments of slab s+1 (complete since the barrier of step s-1) into the other set,
  //   widens the codes of slab s+2 (requested in step s-2, landed by the wait of step s-1) into stage (u+2) % 4,
  //   requests the codes of slab s+4 into the registers just freed.
  // The wait at its end lets this step's own NV loads stay in flight and nothing older: the A loads
  // of slab s+2 (issued in step s-1) have landed, and with the barrier slab s+2 is complete.
  // A 16 x 16 x 32 MFMA keeps the matrix pipe busy for 16 cycles and the wavefront can issue for
  // 12 of them: the other work of a step is cut into pieces of one or two instructions, one piece
  // behind each MFMA, and a scheduling barrier after every such slot keeps it there. Work that is
  // clumped between groups of MFMAs leaves the matrix pipe idle while it issues (measured: 1640
  // cycles per step against 1060 for the MFMAs alone).
  constexpr int S = TN * TM;  // MFMA slots of a step
  constexpr int NR = TM + TN;
  constexpr int NL = NS + NQ;  // scale and code loads
  auto at = [](int i, int n, int lo, int hi) constexpr { return lo + (i * (hi - lo)) / n; };
  constexpr int L0 = 3 * S / 4;  // first slot of the code loads: the last conversion piece sits in the slot before
  static_assert(S >= 4 && S % 4 == 0, "a step has at least four MFMA slots");
  int next_a_off = a_offset(3), next_q_off = q_offset(4), next_s_off = scale_offset(4);
  auto step = [&](auto u_tag, int s) __attribute__((always_inline)) {
    constexpr int u = decltype(u_tag)::value;
    constexpr int par = u & 1;
    // this step's load offsets were computed behind MFMAs of the step before
    const int a_off = next_a_off, q_off = next_q_off, s_off = next_s_off;
    static_for<S>([&](auto q_tag) __attribute__((always_inline)) {
      constexpr int q = decltype(q_tag)::value;
      constexpr int t = q / TM, j = q % TM;
      mfma16<DT>(acc[t][j], wf[par][t], xf[par][j]);
      if constexpr (q == 0) merge_scales(par);
      static_for<NR>([&](auto r_tag) __attribute__((always_inline)) {
        constexpr int r = decltype(r_tag)::value;
        if constexpr (q == at(r, NR, 0, S / 2)) read_fragment(par ^ 1, (u + 1) & 3, r);
      });
      static_for<A_LD>([&](auto i_tag) __attribute__((always_inline)) {
        constexpr int i = decltype(i_tag)::value;
        if constexpr (q == at(i, A_LD, 0, S / 2)) dma_a_pass((u + 3) & 3, a_off, i);
      });
      static_for<NROWS>([&](auto p_tag) __attribute__((always_inline)) {
        constexpr int pp = decltype(p_tag)::value;
        if constexpr (NAT && q == at(pp, NROWS, S / 4, S / 2)) transpose_piece(par, pp);
      });
      constexpr int WD = NAT ? DPC : 4;  // widening pieces (dwords) per unit
      static_for<WD * UNITS>([&](auto p_tag) __attribute__((always_inline)) {
        constexpr int pp = decltype(p_tag)::value;
        if constexpr (q == at(pp, WD * UNITS, S / 2, 3 * S / 4)) widen_piece(par, pp / WD, pp % WD);
        if constexpr (pp % WD == WD - 1 && q == (at(pp, WD * UNITS, S / 2, 3 * S / 4) + 1 < S ? at(pp, WD * UNITS, S / 2, 3 * S / 4) + 1 : S - 1)) store_unit((u + 2) & 3, pp / WD);
      });
      static_for<NL>([&](auto l_tag) __attribute__((always_inline)) {
        constexpr int l = decltype(l_tag)::value;
        if constexpr (q == at(l, NL, L0, S)) {
          if constexpr (l < NS) load_scale_piece(par, s_off, l);
          else load_code_piece(par, q_off, l - NS);
        }
      });
      if constexpr (q == L0) load_scalar_scales(par, s + 4);
      // the offsets of the next step's loads, a few instructions each
      if constexpr (q == at(0, 3, S / 2, S)) next_a_off = a_offset(s + 4);
      if constexpr (q == at(1, 3, S / 2, S) && !NAT) next_q_off = q_offset(s + 5);
      if constexpr (q == S - 1 && NAT) q_walk_advance();
      if constexpr (q == at(2, 3, S / 2, S) && NS > 0) next_s_off = scale_offset(s + 5);
      __builtin_amdgcn_sched_barrier(0);
    });
    __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(NV));
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
  };

  // prologue: slabs 0 and 1 complete, the A loads of slab 2 done, the codes of slabs 2 and 3 in
  // registers, the fragments of slab 0 in set 0
  dma_a(0, 0);
  dma_a(1, 1);
  dma_a(2, 2);
  load_slab(0, 0);
  load_slab(1, 1);
  // The accumulators are cleared while the first loads are on their way: each one goes through an
  // empty statement that pins its register writes here (left alone, the compiler sinks them to
  // just in front of the loop, behind the waits).
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};
      asm volatile("" : "+a"(acc[i][j]));
    }
  __builtin_amdgcn_sched_barrier(0);
  // The optimizer takes the result of a load statement for ready where the statement stands: nothing
  // that reads it may move above the wait (in the steps every slot ends in a scheduling barrier).
  __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));
  __builtin_amdgcn_sched_barrier(0);
  commit_all(0, 0);
  commit_all(1, 1);
  __builtin_amdgcn_sched_barrier(0);
  load_slab(0, 2);
  load_slab(1, 3);
  __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));
  __builtin_amdgcn_sched_barrier(0);
  __syncthreads();
#pragma unroll
  for (int r = 0; r < NR; ++r) read_fragment(0, 0, r);
  __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));
  __builtin_amdgcn_sched_barrier(0);

  for (int s = 0; s < steps; s += 4) {
    step(std::integral_constant<int, 0>{}, s);
    step(std::integral_constant<int, 1>{}, s + 1);
    step(std::integral_constant<int, 2>{}, s + 2);
    step(std::integral_constant<int, 3>{}, s + 3);
  }
  // The loads of the padded slabs are still in flight. Those to LDS must land before the epilogue
  // stages rows there; those to registers must land before the registers are used for anything
  // else: to the compiler their results were ready where the load statements stand and are dead
  // by now, so it would hand the registers to the epilogue at once and the late data would land
  // on top of accumulator values. Naming them after the wait keeps them allocated until then.
  __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int b = 0; b < 2; ++b) {
#pragma unroll
    for (int i = 0; i < (NAT ? NROWS : 2 * UNITS); ++i) asm volatile("" ::"v"(raw[b][i]));
#pragma unroll
    for (int i = 0; i < (kHalfRows ? 4 : NS ? NS : 1); ++i) asm volatile("" ::"v"(sraw[b][i]));
    if constexpr (kRowScalars) asm volatile("" ::"s"(scr[b]));
  }
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  // The MFMAs are opaque statements: nothing tells the compiler that their results take time. The
  // epilogues read every accumulator element with an opaque statement of its own, which stays
  // behind the wait above in program order.
  __builtin_amdgcn_sched_barrier(0);

  // the epilogue stages rows through LDS: half a ring per wavefront
  static_assert(STAGES * A_STAGE / 2 >= staged_rows_bytes(WTN) && STAGES * B_STAGE / 2 >= staged_rows_bytes(WTN), "staging room");
  uint8_t* bufs[4] = {a_ring, a_ring + STAGES * A_STAGE / 2, b_ring, b_ring + STAGES * B_STAGE / 2};
  if constexpr (MODE == kWoFwd)
    store_tile<BM, BN, DT, 1>(acc, 1.0f, nullptr, static_cast<const float*>(scale_ptr), bias, C, M, NO, m0, n0, bufs[0], bufs[1], bufs[2], bufs[3]);
  else if constexpr (MODE == kWoDgradT)
    store_tile<BM, BN, DT, 0>(acc, 1.0f, nullptr, nullptr, nullptr, C, M, NO, m0, n0, bufs[0], bufs[1], bufs[2], bufs[3]);
  else
    store_tile_by_fours<BM, BN, DT>(acc, C, M, NO, m0, n0, bufs[0], bufs[1], bufs[2], bufs[3]);
}

template <int BM, int BN, int DT, int QF, int MODE, int SK>
inline int launch_wo(const void* a, const void* q, const void* scale, int scale_ld, const void* bias, void* c, int M, int NO,
                     int KC, hipStream_t st, int tn_first = 0, int tn_count = -1) {
  if (tn_count < 0) tn_count = (NO + BN - 1) / BN - tn_first;  // to the last tile column
  if (tn_count <= 0) return KM_OK;  // nothing left (a window that starts past the last, narrower tile column)
  const int tiles = ((M + BM - 1) / BM) * tn_count;
  hipLaunchKernelGGL((wo_gemm_kernel<BM, BN, DT, QF, MODE, SK>), dim3(tiles), dim3(256), 0, st, (const uint16_t*)a,
                     (const uint8_t*)q, scale, scale_ld, (const uint16_t*)bias, (uint16_t*)c, M, NO, KC, tn_first, tn_count);
  return km_check_launch("km_wo_gemm");
}

// compute units of the current device (asked once per device; not a stream operation)
inline int compute_units() {
  static int cached[64] = {};
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  if (cached[dev] == 0 && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess) cached[dev] = n;
  return cached[dev];
}

template <int DT, int QF, int MODE, int SK>
inline int launch_config(int config, const void* a, const void* q, const void* scale, int scale_ld, const void* bias, void* c,
                         int M, int NO, int KC, hipStream_t st) {
  switch (config) {
    case 0: return launch_wo<256, 256, DT, QF, MODE, SK>(a, q, scale, scale_ld, bias, c, M, NO, KC, st);
    case 1: return launch_wo<128, 256, DT, QF, MODE, SK>(a, q, scale, scale_ld, bias, c, M, NO, KC, st);
    case 2: return launch_wo<256, 128, DT, QF, MODE, SK>(a, q, scale, scale_ld, bias, c, M, NO, KC, st);
    case 3: return launch_wo<128, 128, DT, QF, MODE, SK>(a, q, scale, scale_ld, bias, c, M, NO, KC, st);
    case 4: return launch_wo<64, 128, DT, QF, MODE, SK>(a, q, scale, scale_ld, bias, c, M, NO, KC, st);
    case 5:
      // 192 columns: whole waves of tiles where 256-column tiles leave compute units idle (3072
      // output columns: 16 x 16 = 256 tiles against 16 x 12 = 192 at M = 4096, 32 x 16 = 512 against
      // 32 x 12 = 384 at M = 8192)
      return launch_wo<256, 192, DT, QF, MODE, SK>(a, q, scale, scale_ld, bias, c, M, NO, KC, st);
    case 6: {
      // 256 x 256 tiles over as many tile columns as fill whole rounds of the card (one tile per
      // compute unit and round), half-size tiles over the rest: the last, partly empty round of large
      // tiles becomes a full round of tiles that take less time (8192 x 3072 outputs: 384 large tiles
      // are one round and a half, so two; 256 large and 256 half tiles are one round each). The half
      // tile is the one whose step costs least in the mode: 256 x 128 where the codes are read as
      // stored with a scale per row (its lanes split the rows of a slab), 128 x 256 otherwise. Every
      // output element is the same sum in the same order as in the other configurations.
      const int tm = (M + 255) / 256, tn = (NO + 255) / 256, cus = compute_units();
      if (cus <= 0) return km_fail(KM_ERR_LAUNCH, "km_wo_gemm: cannot ask for the number of compute units");
      const int whole_cols = whole_round_columns(tm, tn, cus);
      int rc = launch_wo<256, 256, DT, QF, MODE, SK>(a, q, scale, scale_ld, bias, c, M, NO, KC, st, 0, whole_cols);
      if (rc != KM_OK) return rc;
      if constexpr (MODE == kWoDgradN && SK == KM_WSCALE_ROWS)
        return launch_wo<256, 128, DT, QF, MODE, SK>(a, q, scale, scale_ld, bias, c, M, NO, KC, st, 2 * whole_cols, -1);
      else
        return launch_wo<128, 256, DT, QF, MODE, SK>(a, q, scale, scale_ld, bias, c, M, NO, KC, st, whole_cols, -1);
    }
  }
  return km_fail(KM_ERR_ARG, "km_wo_gemm: unknown config");
}

}  // namespace km
