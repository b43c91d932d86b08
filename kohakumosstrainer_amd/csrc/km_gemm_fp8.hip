// fp8 GEMMs for gfx950 on the block-scaled MFMA (V_MFMA_SCALE_F32_16X16X128_F8F6F4):
//
//   C[M,N] = A[M,K] B[N,K]^T (+ bias), A and B e4m3fn with K contiguous, fp32 accumulation
//   over all of K, scales applied in fp32 by the MFMA (mx) or on the accumulator (tensor),
//   bias added in fp32, one rounding at the store.
//
// Replaces the reference's Triton GEMMs (src/kohakumoss_kernels/backends/triton/fp8/gemm.py:
// _dot_scaled_kernel :137-171 and _promote_kernel :108-134 for mx, _scaled_kernel :66-105 for
// the per-tensor recipe; the shared epilogue _store :40-49).
//
// Shape of the kernel. A workgroup of four wavefronts owns a BM x BN tile of C and walks K in
// steps of 128 bytes. Per step the A (BM x 128 B) and B (BN x 128 B) slabs live in two pairs
// of static LDS buffers, filled by direct-to-LDS buffer loads (no staging registers). The A
// fragments of a step are read into registers during the last MFMA group of the step before,
// so an A buffer is free a whole step early: at the top of step k the loads of B(k+1) and then
// of A(k+2) are issued, and just before the last MFMA group of step k the wavefront waits
// only for B(k+1) (vmcnt counts in order), passes the barrier and reads the first fragments of
// step k+1. The A(k+2) loads stay in flight across that barrier, so the fetch stream never
// drains and the MFMA pipe has work across the step boundary. Each wavefront computes a (BM/2) x (BN/2) sub-tile as 16x16 MFMA tiles. The
// MFMA's "A" operand (rows of the 16x16 result) is fed from B (output columns n) and its "B"
// operand from A (tokens m), so a lane ends up with 4 consecutive n of one m and stores 8
// bytes of bf16. Rows past M / N are fetched through buffer descriptors whose range check
// returns zeros.
//
// Operand layout of the 16x16x128 MFMA (measured on gfx950 with one-hot operands): lane l
// carries, for row l%16 and g = l/16, the 16 K bytes [16g, 16g+16) in its first four
// registers and [64+16g, 64+16g+16) in its last four; the E8M0 byte of lane l scales K block
// g (bytes [32g, 32g+32)) of row l%16, whichever lanes hold those bytes. The four block
// scales of a row for one K step are one aligned dword of the natural [rows, K/32] matrix; a
// lane shifts it right by 8*(l/16) so that byte 0 is the scale it must supply. The faster
// path reads the MFMA-packed copy (km_scale_pack_offset): for every K step and group of 128
// rows, 512 bytes ordered [row%16][block][tile=row%128/16], so lane l finds the scale bytes
// of all eight 16-row tiles of its wave in 8 consecutive bytes at 32*(l%16) + 8*(l/16) and
// a wavefront fetches them with one coalesced 512-byte load; op_sel then picks the tile.
//
// LDS layout of a slab: rows of 128 B = 8 chunks of 16 B. Rows r and r+8 of each group of 16
// share one 256-byte line (low / high half) and chunk c of row r sits in slot c ^ (r & 7), so
// the fragment reads (16 lanes = 16 rows at one chunk) touch every bank once. A direct-to-LDS
// load writes lane i of a wavefront at base + 16*i, so the swizzle is applied on the global
// side: lane i fetches the chunk whose slot is i & 7.
#include <stdio.h>

#include <mutex>
#include <vector>

#include "km_gemm_common.h"

namespace km {

// c += A(16x128) * B(128x16) with block scales, accumulating in place: the accumulator is an
// AGPR tuple tied as input and output ("+a"), which keeps all 64 tiles of a wavefront resident
// in the 256 AGPRs with no copies. op_sel picks which byte of each scale register is used
// (tile index % 4); it is an immediate, hence one statement per combination.
// ZERO: c = A * B, the form of a tile's first K step: the accumulator is written without being
// read, so it needs no clearing and carries nothing from one tile of a work-group to the next.
#define KM_MFMA_ASM(OSA, OSB, OHA, OHB)                                                              \
  do {                                                                                                \
    if constexpr (ZERO)                                                                               \
      asm("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, 0, %3, %4 op_sel:[" #OSA "," #OSB ",0] op_sel_hi:[" #OHA "," #OHB ",0]" \
          : "=a"(c)                                                                                   \
          : "v"(a), "v"(b), "v"(sa), "v"(sb));                                                        \
    else                                                                                              \
      asm("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:[" #OSA "," #OSB ",0] op_sel_hi:[" #OHA "," #OHB ",0]" \
          : "+a"(c)                                                                                   \
          : "v"(a), "v"(b), "v"(sa), "v"(sb));                                                        \
  } while (0)
template <int SEL_A, int SEL_B, bool ZERO = false>
__device__ __forceinline__ void mfma_acc(v4f& c, const v8i& a, const v8i& b, int sa, int sb) {
  constexpr int code = (SEL_A & 3) * 4 + (SEL_B & 3);
  if constexpr (code == 0) KM_MFMA_ASM(0, 0, 0, 0);
  else if constexpr (code == 1) KM_MFMA_ASM(0, 1, 0, 0);
  else if constexpr (code == 2) KM_MFMA_ASM(0, 0, 0, 1);
  else if constexpr (code == 3) KM_MFMA_ASM(0, 1, 0, 1);
  else if constexpr (code == 4) KM_MFMA_ASM(1, 0, 0, 0);
  else if constexpr (code == 5) KM_MFMA_ASM(1, 1, 0, 0);
  else if constexpr (code == 6) KM_MFMA_ASM(1, 0, 0, 1);
  else if constexpr (code == 7) KM_MFMA_ASM(1, 1, 0, 1);
  else if constexpr (code == 8) KM_MFMA_ASM(0, 0, 1, 0);
  else if constexpr (code == 9) KM_MFMA_ASM(0, 1, 1, 0);
  else if constexpr (code == 10) KM_MFMA_ASM(0, 0, 1, 1);
  else if constexpr (code == 11) KM_MFMA_ASM(0, 1, 1, 1);
  else if constexpr (code == 12) KM_MFMA_ASM(1, 0, 1, 0);
  else if constexpr (code == 13) KM_MFMA_ASM(1, 1, 1, 0);
  else if constexpr (code == 14) KM_MFMA_ASM(1, 0, 1, 1);
  else KM_MFMA_ASM(1, 1, 1, 1);
}
#undef KM_MFMA_ASM

// a (uniform) buffer descriptor, in scalar registers wherever the compiler has put it
__device__ __forceinline__ v4i scalar_rsrc(const v4i& a) {
  return v4i{__builtin_amdgcn_readfirstlane(a.x), __builtin_amdgcn_readfirstlane(a.y), __builtin_amdgcn_readfirstlane(a.z), __builtin_amdgcn_readfirstlane(a.w)};
}
// one of two buffer descriptors by a uniform condition, kept in scalar registers
__device__ __forceinline__ v4i pick_rsrc(bool first, const v4i& a, const v4i& b) {
  return v4i{__builtin_amdgcn_readfirstlane(first ? a.x : b.x), __builtin_amdgcn_readfirstlane(first ? a.y : b.y),
             __builtin_amdgcn_readfirstlane(first ? a.z : b.z), __builtin_amdgcn_readfirstlane(first ? a.w : b.w)};
}

// c += A(16x64) * B(64x16) of int8 codes with int32 accumulation (V_MFMA_I32_16X16X64_I8), the
// accumulator tied in AGPRs as above (its registers hold int32 bits). Lane l supplies 16
// consecutive K bytes of row l%16 in both operands, so each 16-byte half of a 128-byte-step
// fragment (K bytes [16g, 16g+16) and [64+16g, 64+16g+16)) feeds one instruction: two of them
// cover the step, in a K order that is the same for both operands.
template <bool HI, bool ZERO = false>
__device__ __forceinline__ void mfma_i8_half(v4f& c, const v8i& a, const v8i& b) {
  const v4i ah = HI ? __builtin_shufflevector(a, a, 4, 5, 6, 7) : __builtin_shufflevector(a, a, 0, 1, 2, 3);
  const v4i bh = HI ? __builtin_shufflevector(b, b, 4, 5, 6, 7) : __builtin_shufflevector(b, b, 0, 1, 2, 3);
  if constexpr (ZERO) asm("v_mfma_i32_16x16x64_i8 %0, %1, %2, 0" : "=a"(c) : "v"(ah), "v"(bh));
  else asm("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(c) : "v"(ah), "v"(bh));
}

// A1: one A buffer instead of two (the A slab of step k+1 is requested at the top of step k,
// once every wavefront holds the fragments of step k in registers, and waited for at its end).
// Nothing stays in flight across the step boundary then, but the tile needs 3/4 of the LDS and,
// with half the accumulators of the largest tile, two workgroups share a compute unit and fill
// each other's waits, prologue and epilogue.
// I8: int8 codes on the int32 MFMA (no block scales), scale vectors applied in the reference's
// order of roundings at the store.
// B3: a third B buffer (the whole 160 KiB of LDS). Every fetch of a step (A, B, and the scale lines
// as a touch that only fills L2) is issued two steps before its use instead of one for B and the
// scales: a load that misses the XCD's L2 takes longer than one step to arrive.
template <int BM, int BN, bool MX, bool SCALE_KM, int OUT, bool A1, bool I8, bool B3 = false>
__global__ __launch_bounds__(256, A1 ? 2 : 1) void gemm_fp8_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ As, const uint8_t* __restrict__ B,
    const uint8_t* __restrict__ Bs, const float* __restrict__ sa, const float* __restrict__ sb,
    const uint16_t* __restrict__ bias, uint16_t* __restrict__ C, int M, int N, int K, int scale_vectors) {
  constexpr int NT = 256;
  constexpr int WTM = BM / 2, WTN = BN / 2;
  constexpr int TM = WTM / 16, TN = WTN / 16;
  constexpr int A_BYTES = BM * kStepBytes, B_BYTES = BN * kStepBytes;
  constexpr int A_LD = BM / 32, B_LD = BN / 32;  // 32 rows (4 KiB) per pass of 256 lanes
  static_assert(!(A1 && B3), "the third B buffer goes with two A buffers");
  constexpr int kTouches = (B3 && MX && SCALE_KM) ? 2 : 0;
  // loads of this step that may still be in flight at its end: A1 none, else the A passes (and, B3, the
  // B passes and scale touches, all issued after the step's own scale fetch)
  constexpr int kWaitAllButA = wait_vm_lgkm0(A1 ? 0 : B3 ? A_LD + B_LD + kTouches : A_LD);
  static_assert(BM % 32 == 0 && BN % 32 == 0 && TM >= 1 && TN >= 2, "tile");
  static_assert(TM * (TN - 1) >= BM / 32 + BN / 32, "every fetch pass needs its own MFMA slot");
  __shared__ __attribute__((aligned(1024))) uint8_t a_buf0[A_BYTES];
  __shared__ __attribute__((aligned(1024))) uint8_t a_buf1[A1 ? 16 : A_BYTES];
  __shared__ __attribute__((aligned(1024))) uint8_t b_buf0[B_BYTES];
  __shared__ __attribute__((aligned(1024))) uint8_t b_buf1[B_BYTES];
  __shared__ __attribute__((aligned(1024))) uint8_t b_buf2[B3 ? B_BYTES : 16];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = (wave >> 1) * WTM, wn = (wave & 1) * WTN;
  const int r16 = lane & 15, g = lane >> 4;
  const int nk = K / kStepBytes;
  const int kb = K >> 5;  // scale bytes per row (natural layout)
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const int total_tiles = tiles_m * tiles_n;

  // staging map of a pass: 8 lanes per row; 16 lanes cover rows r and r+8 (one LDS line)
  const int w = tid >> 3;
  const int srow = ((w >> 4) << 4) + ((w & 1) << 3) + ((w >> 1) & 7);  // 0 .. 31
  const int src_chunk = (tid & 7) ^ (srow & 7);
  const int ld_voff = srow * K + src_chunk * 16;
  const int pass_stride = 32 * K;

  // What depends on the tile: the work-group walks the tiles pid, pid + gridDim.x, ...
  int m0 = 0, n0 = 0;
  // buffer descriptors start at the tile's first row; their range check (on the per-lane
  // offset) turns rows past the end into zeros
  v4i a_rsrc, b_rsrc;
  // scales: MFMA rows come from B (n), MFMA columns from A (m)
  v4i ws_rsrc, xs_rsrc;
  int ws_off[SCALE_KM ? 1 : TN], xs_off[SCALE_KM ? 1 : TM];
  int ws_base = 0, xs_base = 0, ws_sel = 0, xs_sel = 0;
  const int rbn = (N + 127) >> 7, rbm = (M + 127) >> 7;  // packed scales: 128-row blocks
  const int ws_step = SCALE_KM ? rbn * 512 : 4, xs_step = SCALE_KM ? rbm * 512 : 4;
  if constexpr (MX && SCALE_KM) {
    // packed: byte offset ((ks*RB + r/128)*16 + r%16)*32 + 8*block + (r%128)/16
    ws_rsrc = raw_rsrc(Bs, (uint32_t)min((int64_t)nk * rbn * 512, (int64_t)0x7FFFFFFF));
    xs_rsrc = raw_rsrc(As, (uint32_t)min((int64_t)nk * rbm * 512, (int64_t)0x7FFFFFFF));
    ws_off[0] = r16 * 32 + g * 8;
    xs_off[0] = ws_off[0];
  }
  // the part of it that a work-group needs of its next tile while it finishes one (see kSeamless)
  auto tile_operands = [&](int pid, int& tm0, int& tn0, v4i& ta, v4i& tb, int& tws_base, int& txs_base, int& tws_sel, int& txs_sel)
                           __attribute__((always_inline)) {
    int tile_m, tile_n;
    tile_of(pid, tiles_m, tiles_n, tile_m, tile_n);
    tm0 = tile_m * BM;
    tn0 = tile_n * BN;
    ta = raw_rsrc(A + (size_t)tm0 * K, (uint32_t)min((int64_t)(M - tm0) * K, (int64_t)0x7FFFFFFF));
    tb = raw_rsrc(B + (size_t)tn0 * K, (uint32_t)min((int64_t)(N - tn0) * K, (int64_t)0x7FFFFFFF));
    if constexpr (MX && SCALE_KM) {
      tws_base = min((tn0 + wn) >> 7, rbn - 1) * 512;  // waves wholly past the edge read valid bytes
      txs_base = min((tm0 + wm) >> 7, rbm - 1) * 512;
      tws_sel = (((tn0 + wn) & 127) >> 4) * 8;  // bit shift to this wave's first tile
      txs_sel = (((tm0 + wm) & 127) >> 4) * 8;
    }
  };
  auto set_tile = [&](int pid) __attribute__((always_inline)) {
    tile_operands(pid, m0, n0, a_rsrc, b_rsrc, ws_base, xs_base, ws_sel, xs_sel);
    if constexpr (MX && !SCALE_KM) {
      // natural [rows, K/32]; row indices are clamped to the last valid row
      ws_rsrc = raw_rsrc(Bs + (size_t)n0 * kb, (uint32_t)min((int64_t)(N - n0) * kb, (int64_t)0x7FFFFFFF));
      xs_rsrc = raw_rsrc(As + (size_t)m0 * kb, (uint32_t)min((int64_t)(M - m0) * kb, (int64_t)0x7FFFFFFF));
#pragma unroll
      for (int t = 0; t < TN; ++t) ws_off[t] = min(wn + t * 16 + r16, N - 1 - n0) * kb;
#pragma unroll
      for (int t = 0; t < TM; ++t) xs_off[t] = min(wm + t * 16 + r16, M - 1 - m0) * kb;
    }
  };
  int pid = blockIdx.x;
  set_tile(pid);
  int nm0 = m0, nn0 = n0, nws_base = ws_base, nxs_base = xs_base, nws_sel = ws_sel, nxs_sel = xs_sel;
  v4i na_rsrc = a_rsrc, nb_rsrc = b_rsrc;

  v4f acc[TN][TM];

  v8i xf[TM];
  v8i wcur;
  // Scale operands of the step being multiplied / raw words of the next step in flight.
  // Packed layout: two registers per operand hold the bytes of tiles 0-3 and 4-7 (op_sel picks
  // one); natural layout: one register per tile, its byte 0 is the scale.
  constexpr int WS = SCALE_KM ? 2 : TN, XS = SCALE_KM ? 2 : TM;
  // Two sets, one per step parity: a step reads its own set while the next step's set is
  // written, so no scale register is overwritten while an MFMA that reads it is in flight
  // (the inline-asm MFMAs are opaque to the compiler's hazard handling).
  int wscale[2][WS], xscale[2][XS];
  uint32_t wraw[WS], xraw[XS];
  uint64_t wraw64 = 0, xraw64 = 0;  // packed layout: the 8 scale bytes of a lane
  // A 96-row wavefront (192-row tiles) may start 64 or 96 rows into a 128-row scale block: its
  // tiles then continue in the next block, whose 8 bytes are fetched as well.
  constexpr bool kWStraddle = MX && SCALE_KM && WTN % 64 != 0, kXStraddle = MX && SCALE_KM && WTM % 64 != 0;
  uint64_t wraw64b = 0, xraw64b = 0;

  // one 4 KiB pass (32 rows) of a slab: each wavefront moves 1 KiB with one instruction
  // LDS buffers are named by their LDS byte address (uniform 32-bit values): the B buffers of the
  // three-buffer variant change roles from step to step
  auto dma_pass = [&](const v4i& rsrc, uint32_t buf, int koff, int i, int beyond = 0) __attribute__((always_inline)) {
    hidden_dma_b128(scalar_rsrc(rsrc), buf + i * 4096 + wave * 1024, ld_voff + i * pass_stride + beyond, koff);
  };
  // inside the K loop: every SGPR these read is loop invariant or comes from the scalar ALU.
  // `beyond` (0 or 2^31) pushes the per-lane offset past the descriptor's range: the pass then
  // fills its LDS rows with zeros
  auto loop_dma_pass = [&](const v4i& rsrc, uint32_t buf, int koff, int i, int beyond = 0) __attribute__((always_inline)) {
    loop_dma_b128(rsrc, buf + i * 4096 + wave * 1024, ld_voff + i * pass_stride + beyond, koff);
  };
  auto dma_a = [&](uint32_t buf, int ks) __attribute__((always_inline)) {
    const int koff = __builtin_amdgcn_readfirstlane(ks * kStepBytes);
#pragma unroll
    for (int i = 0; i < A_LD; ++i) dma_pass(a_rsrc, buf, koff, i);
  };
  auto dma_b = [&](uint32_t buf, int ks, int beyond = 0) __attribute__((always_inline)) {
    const int koff = __builtin_amdgcn_readfirstlane(ks * kStepBytes);
#pragma unroll
    for (int i = 0; i < B_LD; ++i) dma_pass(b_rsrc, buf, koff, i, beyond);
  };
  // B3: the 2 x 512 scale bytes this wavefront will fetch for step ks, requested early so that the
  // fetch finds them in L2; the 2 x 256 bytes land in the first bytes of `scratch`'s pass 0 slot of
  // this wavefront, which its own B pass 0 (issued later, so arriving later) overwrites
  auto scale_touch = [&](int ks, uint32_t scratch) __attribute__((always_inline)) {
    if constexpr (kTouches > 0) {
      const int wso = __builtin_amdgcn_readfirstlane(ks * ws_step + ws_base);
      const int xso = __builtin_amdgcn_readfirstlane(ks * xs_step + xs_base);
      hidden_touch_b32(scalar_rsrc(ws_rsrc), scratch + wave * 1024, ws_off[0], wso);
      hidden_touch_b32(scalar_rsrc(xs_rsrc), scratch + wave * 1024 + 256, xs_off[0], xso);
    }
  };
  // `wbase`, `xbase`: ws_base and xs_base of the tile the step belongs to
  auto scale_fetch = [&](int ks, int wbase, int xbase) __attribute__((always_inline)) {
    if constexpr (MX) {
      const int wso = __builtin_amdgcn_readfirstlane(ks * ws_step + wbase);
      const int xso = __builtin_amdgcn_readfirstlane(ks * xs_step + xbase);
      // (descriptors that are set anew for every tile come out of the tile loop's merge as vector
      // registers; the loads' five wait states cover the lane read that moves them back)
      const v4i wr = scalar_rsrc(ws_rsrc), xr = scalar_rsrc(xs_rsrc);
      if constexpr (SCALE_KM) {
        wraw64 = hidden_load_b64(wr, ws_off[0], wso);
        xraw64 = hidden_load_b64(xr, xs_off[0], xso);
        // the next 128-row block of the same step, clamped to the last one
        if constexpr (kWStraddle) wraw64b = hidden_load_b64(wr, ws_off[0], __builtin_amdgcn_readfirstlane(ks * ws_step + min(wbase + 512, (rbn - 1) * 512)));
        if constexpr (kXStraddle) xraw64b = hidden_load_b64(xr, xs_off[0], __builtin_amdgcn_readfirstlane(ks * xs_step + min(xbase + 512, (rbm - 1) * 512)));
      } else {
#pragma unroll
        for (int t = 0; t < TN; ++t)
          wraw[t] = hidden_load_b32(wr, ws_off[t], wso);
#pragma unroll
        for (int t = 0; t < TM; ++t)
          xraw[t] = hidden_load_b32(xr, xs_off[t], xso);
      }
    }
  };
  // `live` is all ones for a real step and zero for the padding step of an odd step count:
  // zero scale bytes (2^-127 on both sides) make that step add exactly 0. `wsel`, `xsel`:
  // ws_sel and xs_sel of the tile the fetched bytes belong to.
  auto scale_commit = [&](auto set_tag, uint32_t live, int wsel, int xsel) __attribute__((always_inline)) {
    constexpr int P = decltype(set_tag)::value;
    if constexpr (!MX) {
#pragma unroll
      for (int t = 0; t < WS; ++t) wscale[P][t] = (int)(0x7F7F7F7Fu & live);
#pragma unroll
      for (int t = 0; t < XS; ++t) xscale[P][t] = (int)(0x7F7F7F7Fu & live);
    } else if constexpr (SCALE_KM) {
      uint64_t wv = wraw64 >> wsel;
      uint64_t xv = xraw64 >> xsel;
      if constexpr (kWStraddle) wv |= wsel ? wraw64b << (64 - wsel) : 0;
      if constexpr (kXStraddle) xv |= xsel ? xraw64b << (64 - xsel) : 0;
      wscale[P][0] = (int)((uint32_t)wv & live); wscale[P][1] = (int)((uint32_t)(wv >> 32) & live);
      xscale[P][0] = (int)((uint32_t)xv & live); xscale[P][1] = (int)((uint32_t)(xv >> 32) & live);
    } else {
#pragma unroll
      for (int t = 0; t < TN; ++t) wscale[P][t] = (int)((wraw[t] >> (8 * g)) & live);
#pragma unroll
      for (int t = 0; t < TM; ++t) xscale[P][t] = (int)((xraw[t] >> (8 * g)) & live);
    }
  };
  typedef __attribute__((address_space(3))) const v4i* lds_v4i_cptr;
  auto fragment = [&](uint32_t slab, int row) __attribute__((always_inline)) -> v8i {
    const v4i lo = *(lds_v4i_cptr)(slab + slab_offset(row, g));
    const v4i hi = *(lds_v4i_cptr)(slab + slab_offset(row, g + 4));
    return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };
  // two steps per trip, one per buffer parity; an odd step count is padded with a zero-scaled
  // step (int8: a step whose B slab is zeros)
  const int nsteps = (nk + 1) & ~1;
  // The K loops of a work-group's tiles form one pipeline (not with the third B buffer, whose
  // roles do not come round after an even number of steps; not with natural-layout scales, whose
  // per-lane offsets depend on the tile; not with the single A buffer, where two work-groups share
  // a compute unit's registers and the first fragments of the next tile would not fit beside the
  // epilogue's): a fetch for slab s >= nsteps is
  // slab s - nsteps of the next tile, and it lands in the buffer where that tile expects it,
  // because nsteps is even. So the last steps of a tile already fetch the first slabs and scales
  // of the next and read its first fragments, and between two tiles there is only the epilogue.
  // `more`: this work-group has another tile (else such fetches repeat the tile's last slab).
  constexpr bool kSeamless = !B3 && !A1 && (SCALE_KM || !MX);
  bool more = false;
  // One K step with parity P: A(k) is already in registers, B(k) is in b_cur. Fetches B(k+1)
  // into b_nxt (free since the barrier in the last group of the step before) and A(k+2) into
  // a_cur (its A(k) was consumed during the step before; a barrier just ahead of the first A
  // pass makes sure by every wavefront), multiplies, waits for B(k+1) only,
  // and reads the first fragments of step k+1 (A(k+1) from a_nxt was issued a step earlier)
  // during the last MFMA group; each fragment register is reloaded one MFMA after the last
  // MFMA that read it. The scales of step k+1 are committed to set P^1.
  //
  // The fetch instructions are spread between the MFMAs of the first TN-1 groups (B passes
  // over the first third, A passes over the rest): a wavefront that queues them back to back
  // blocks on the address unit it shares with the other three and issues no MFMA meanwhile.
  constexpr int kWindow = TM * (TN - 1);           // MFMAs before the last group
  // (B3: both are needed two steps on, so the window is shared in proportion)
  constexpr int kBWindow = B3 ? kWindow * B_LD / (A_LD + B_LD) : kWindow / 3 > B_LD ? kWindow / 3 : B_LD;
  // b_fill: the buffer this step's B passes write, B(k+1) into b_nxt without B3, B(k+2) into the
  // third buffer with it (free since the barrier at the end of step k-1, whose b_cur it was)
  constexpr int kBAhead = B3 ? 2 : 1;
  constexpr int kAAhead = A1 ? 1 : 2;
  auto step = [&](uint32_t a_cur, uint32_t a_nxt, uint32_t b_cur, uint32_t b_nxt, uint32_t b_fill, int ks, auto set_tag, auto first_tag)
                  __attribute__((always_inline)) {
    constexpr int P = decltype(set_tag)::value;
    constexpr bool FIRST = decltype(first_tag)::value;  // the tile's first step writes the accumulators without reading them
    // slab s of this tile, or slab s - nsteps of the next; past the end of the last tile, the last slab again
    const bool wrap = kSeamless && more;
    const bool s_over = wrap && ks + 1 >= nsteps, b_over = wrap && ks + kBAhead >= nsteps, a_over = wrap && ks + kAAhead >= nsteps;
    const int s_next = s_over ? ks + 1 - nsteps : min(ks + 1, nk - 1);
    const int koff_b = __builtin_amdgcn_readfirstlane((b_over ? ks + kBAhead - nsteps : min(ks + kBAhead, nk - 1)) * kStepBytes);
    const int koff_a = __builtin_amdgcn_readfirstlane((a_over ? ks + kAAhead - nsteps : min(ks + kAAhead, nk - 1)) * kStepBytes);
    const v4i b_src = pick_rsrc(b_over, nb_rsrc, b_rsrc);
    const v4i a_src = pick_rsrc(a_over, na_rsrc, a_rsrc);
    // int8 has no scale to zero the padding step of an odd step count with: its B slab is zeros
    const int b_beyond = I8 ? __builtin_amdgcn_readfirstlane(!b_over && ks + kBAhead >= nk ? (int)0x80000000 : 0) : 0;
    if constexpr (B3) scale_fetch(s_next, s_over ? nws_base : ws_base, s_over ? nxs_base : xs_base);  // ahead of the B passes, which may stay in flight
    scale_touch(min(ks + 3, nk - 1), b_fill);
    __builtin_amdgcn_sched_barrier(0);
    static_for<TN>([&](auto t_tag) __attribute__((always_inline)) {
      constexpr int t = decltype(t_tag)::value;
      v8i wnext;
      if constexpr (t + 1 < TN) {
        wnext = fragment(b_cur, wn + (t + 1) * 16 + r16);
      } else {
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(kWaitAllButA);  // B(k+1), scales(k+1) (and A(k+1)) landed
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        wnext = fragment(b_nxt, wn + r16);
      }
      static_for<TM>([&](auto j_tag) __attribute__((always_inline)) {
        constexpr int j = decltype(j_tag)::value;
        constexpr int q = t * TM + j;  // position in the step's MFMA sequence
        // the scales of the next step are requested behind the step's first MFMA, not ahead of it (the four
        // wavefronts' loads queue at the address unit, and at the top of the step nothing runs meanwhile);
        // still ahead of every A pass, so the wait at the step's end covers them
        if constexpr (q == 1 && !B3) {
          __builtin_amdgcn_sched_barrier(0);
          scale_fetch(s_next, s_over ? nws_base : ws_base, s_over ? nxs_base : xs_base);
          __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (I8) {
          // two tiles per pair of slots, low halves then high halves: the two instructions that
          // add into one accumulator are two instructions apart instead of back to back
          static_assert(TM % 2 == 0, "int8 tiles are issued in pairs");
          if constexpr ((j & 1) == 0) {
            mfma_i8_half<false, FIRST>(acc[t][j], wcur, xf[j]);
            mfma_i8_half<false, FIRST>(acc[t][j + 1], wcur, xf[j + 1]);
          } else {
            mfma_i8_half<true>(acc[t][j - 1], wcur, xf[j - 1]);
            mfma_i8_half<true>(acc[t][j], wcur, xf[j]);
          }
        } else if constexpr (SCALE_KM)
          mfma_acc<t, j, FIRST>(acc[t][j], wcur, xf[j], wscale[P][(t >> 2) % WS], xscale[P][(j >> 2) % XS]);
        else
          mfma_acc<0, 0, FIRST>(acc[t][j], wcur, xf[j], wscale[P][t % WS], xscale[P][j % XS]);
        if constexpr (t + 1 < TN) {
          // B pass i goes after MFMA i*kBWindow/B_LD, A pass i after kBWindow + i*(kWindow-kBWindow)/A_LD
          // (A1: everything is needed at the end of this step, so one pass per MFMA from the start)
          static_for<B_LD>([&](auto i_tag) __attribute__((always_inline)) {
            constexpr int i = decltype(i_tag)::value;
            if constexpr (q == (A1 ? i : i * kBWindow / B_LD)) {
              __builtin_amdgcn_sched_barrier(0);
              loop_dma_pass(b_src, b_fill, koff_b, i, b_beyond);
              __builtin_amdgcn_sched_barrier(0);
            }
          });
          static_for<A_LD>([&](auto i_tag) __attribute__((always_inline)) {
            constexpr int i = decltype(i_tag)::value;
            if constexpr (q == (A1 ? B_LD + i : kBWindow + i * (kWindow - kBWindow) / A_LD)) {
              __builtin_amdgcn_sched_barrier(0);
              if constexpr (i == 0) {
                // a_cur still holds A(k): its fragments were read at the end of the step before.
                // Waiting for them here, not at the top of the step, costs nothing: they arrived
                // long ago, and every wavefront must have them before the slab is overwritten.
                __builtin_amdgcn_s_waitcnt(kWaitLgkm0);
                __syncthreads();
              }
              loop_dma_pass(a_src, a_cur, koff_a, i);
              __builtin_amdgcn_sched_barrier(0);
            }
          });
        }
        if constexpr (t + 1 == TN && j >= 1) {
          __builtin_amdgcn_sched_barrier(0);
          xf[j - 1] = fragment(a_nxt, wm + (j - 1) * 16 + r16);
        }
      });
      if constexpr (t + 1 == TN) {
        __builtin_amdgcn_sched_barrier(0);
        xf[TM - 1] = fragment(a_nxt, wm + (TM - 1) * 16 + r16);
      }
      wcur = wnext;
    });
    if constexpr (!I8)
      scale_commit(std::integral_constant<int, P ^ 1>{}, ks + 1 < nk || s_over ? 0xFFFFFFFFu : 0u, s_over ? nws_sel : ws_sel, s_over ? nxs_sel : xs_sel);
    __builtin_amdgcn_sched_barrier(0);
  };
  using set0_t = std::integral_constant<int, 0>;
  using set1_t = std::integral_constant<int, 1>;

  const uint32_t la0 = lds_offset(a_buf0), la1 = A1 ? la0 : lds_offset(a_buf1);
  const uint32_t lb0 = lds_offset(b_buf0), lb1 = lds_offset(b_buf1), lb2 = lds_offset(b_buf2);
  // Prologue of a pipeline: A(0), B(0) (B3: and A(1), B(1)) and the scales of step 0 of the current tile,
  // the first fragments in registers. The second A slab is not needed before the end of step 0,
  // whose closing wait leaves in flight only as many loads as the A passes that step issues
  // itself: requested behind the wait for the first slabs, its passes find the address unit idle.
  auto prologue = [&]() __attribute__((always_inline)) {
    dma_a(la0, 0);
    dma_b(lb0, 0);
    scale_fetch(0, ws_base, xs_base);
    if constexpr (B3) {
      dma_a(la1, min(1, nk - 1));
      dma_b(lb1, min(1, nk - 1), I8 && nk < 2 ? (int)0x80000000 : 0);
      scale_touch(min(1, nk - 1), lb2);
      scale_touch(min(2, nk - 1), lb2);
    }
    __builtin_amdgcn_s_waitcnt(kWaitVm0);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    if constexpr (!A1 && !B3) dma_a(la1, min(1, nk - 1));
    if constexpr (!I8) scale_commit(set0_t{}, 0xFFFFFFFFu, ws_sel, xs_sel);
#pragma unroll
    for (int j = 0; j < TM; ++j) xf[j] = fragment(la0, wm + j * 16 + r16);
    wcur = fragment(lb0, wn + r16);
  };
  prologue();

  for (;;) {
    const int next_pid = pid + (int)gridDim.x;
    more = next_pid < total_tiles;
    if (kSeamless && more) tile_operands(next_pid, nm0, nn0, na_rsrc, nb_rsrc, nws_base, nxs_base, nws_sel, nxs_sel);

    if constexpr (B3) {
      // the three B buffers take the roles (multiplied now, next, being filled) in turn
      uint32_t b_now = lb0, b_next = lb1, b_fill = lb2;
      step(la0, la1, b_now, b_next, b_fill, 0, set0_t{}, std::true_type{});
      step(la1, la0, b_next, b_fill, b_now, 1, set1_t{}, std::false_type{});
      for (int ks = 2; ks < nsteps; ks += 2) {
        const uint32_t was_now = b_now;
        b_now = b_fill;
        b_fill = b_next;
        b_next = was_now;
        step(la0, la1, b_now, b_next, b_fill, ks, set0_t{}, std::false_type{});
        step(la1, la0, b_next, b_fill, b_now, ks + 1, set1_t{}, std::false_type{});
      }
    } else {
      // the first pair of steps stands alone: step 0 writes the accumulators without reading them
      step(la0, la1, lb0, lb1, lb1, 0, set0_t{}, std::true_type{});
      step(la1, la0, lb1, lb0, lb0, 1, set1_t{}, std::false_type{});
      for (int ks = 2; ks < nsteps; ks += 2) {
        step(la0, la1, lb0, lb1, lb1, ks, set0_t{}, std::false_type{});
        step(la1, la0, lb1, lb0, lb0, ks + 1, set1_t{}, std::false_type{});
      }
    }
    // With another tile to go, the loads in flight are its second A slab on its way to the second
    // A buffer and nothing else; the epilogue stages rows in the second B buffer, which every
    // wavefront finished reading before the barrier in the last MFMA group. Otherwise the last
    // (repeated) fetches must be done before the work-group gives up its LDS.
    if (!(kSeamless && more)) __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));

    // The MFMAs above are opaque to the compiler's hazard handling: give the last ones time to
    // retire before the accumulators are read. The epilogue reads every accumulator element with an
    // opaque statement of its own, which stays behind this one.
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
    if constexpr (!kSeamless) __syncthreads();  // every wavefront is done reading fragments

    // epilogue: bias (and the per-tensor scales) on the fp32 accumulator, one rounding
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
    constexpr int kEpilogue = I8 ? 2 : MX ? 0 : 1;
    static_assert(staged_rows_bytes(WTN) <= B_BYTES / 4, "epilogue staging in the quarters of a B buffer");
    store_tile<BM, BN, OUT, kEpilogue, false>(acc, post, row_scale, col_scale, bias, C, M, N, m0, n0, b_buf1, b_buf1 + B_BYTES / 4,
                                              b_buf1 + B_BYTES / 2, b_buf1 + 3 * (B_BYTES / 4));
    if (!more) break;
    pid = next_pid;
    if constexpr (kSeamless) {
      m0 = nm0; n0 = nn0; a_rsrc = na_rsrc; b_rsrc = nb_rsrc;
      ws_base = nws_base; xs_base = nxs_base; ws_sel = nws_sel; xs_sel = nxs_sel;
      // step 0 of the next tile fetches into the second B buffer: every wavefront must have read its rows back
      __syncthreads();
    } else {
      set_tile(pid);
      __syncthreads();
      prologue();
    }
  }
}

struct GemmConfig {
  int bm, bn, b_stages, mfma;  // mfma: rows of the MFMA tile (16: 16x16x128, 32: 32x32x64)
};
// Largest tile first: the host-side table ranks candidates the way the reference ranks its
// Triton tiles (large tiles for large M). Four wavefronts in a 2 x 2 grid each.
static const GemmConfig kGemmConfigs[] = {
    {256, 256, 2, 16},
    {128, 256, 2, 16},
    {256, 128, 2, 16},
    {128, 128, 2, 16},
    {64, 128, 2, 16},
    {256, 256, 3, 16},
    {256, 256, 2, 32},
    {256, 192, 2, 16},
};
constexpr int kNumGemmConfigs = sizeof(kGemmConfigs) / sizeof(kGemmConfigs[0]);

// Work-groups of 256 threads of `kernel` that the current device holds at once (compute units x
// work-groups per unit), asked once per kernel and device. A multiple of the 8 XCDs, so that
// tile pid + grid lands on the XCD of tile pid (tile_of deals tiles to XCDs by pid % 8).
static int resident_workgroups(const void* kernel) {
  struct Entry { const void* kernel; int device; int count; };
  static std::mutex mu;
  static std::vector<Entry> seen;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return -1;
  std::lock_guard<std::mutex> lock(mu);
  for (const Entry& e : seen)
    if (e.kernel == kernel && e.device == device) return e.count;
  int per_cu = 0, cus = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, 0) != hipSuccess) return -1;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) return -1;
  int count = per_cu * cus;
  if (count >= kXcds) count -= count % kXcds;
  if (count <= 0) return -1;
  seen.push_back({kernel, device, count});
  return count;
}

template <int BM, int BN, bool MX, bool SCALE_KM, int OUT, bool A1, bool I8, bool B3 = false>
static int launch_gemm(const void* a, const void* as, const void* b, const void* bs, const float* sa,
                       const float* sb, const void* bias, void* c, int M, int N, int K, int scale_vectors,
                       hipStream_t st) {
  const int tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  // The large tiles (one work-group per compute unit) run as many work-groups as the card holds at
  // once, each walking the tiles pid, pid + grid, ...; the small ones, two work-groups to a
  // compute unit that fill each other's gaps, measured 3-5 % slower that way than with one
  // work-group per tile handed out as compute units fall free.
  int grid = tiles;
  if constexpr (BM >= 256) {
    const int resident = resident_workgroups(reinterpret_cast<const void*>(&gemm_fp8_kernel<BM, BN, MX, SCALE_KM, OUT, A1, I8, B3>));
    if (resident <= 0) return km_fail(KM_ERR_LAUNCH, "km_gemm: occupancy query failed");
    if (resident < tiles) grid = resident;
  }
  hipLaunchKernelGGL((gemm_fp8_kernel<BM, BN, MX, SCALE_KM, OUT, A1, I8, B3>), dim3(grid), dim3(256), 0, st,
                     (const uint8_t*)a, (const uint8_t*)as, (const uint8_t*)b, (const uint8_t*)bs, sa, sb,
                     (const uint16_t*)bias, (uint16_t*)c, M, N, K, scale_vectors);
  return km_check_launch("km_gemm");
}

template <bool MX, bool SCALE_KM, int OUT, bool I8 = false>
static int dispatch_config(int config, const void* a, const void* as, const void* b, const void* bs,
                           const float* sa, const float* sb, const void* bias, void* c, int M, int N,
                           int K, int scale_vectors, hipStream_t st) {
  switch (config) {
    case 0: return launch_gemm<256, 256, MX, SCALE_KM, OUT, false, I8>(a, as, b, bs, sa, sb, bias, c, M, N, K, scale_vectors, st);
    case 1: return launch_gemm<128, 256, MX, SCALE_KM, OUT, true, I8>(a, as, b, bs, sa, sb, bias, c, M, N, K, scale_vectors, st);
    case 2: return launch_gemm<256, 128, MX, SCALE_KM, OUT, false, I8>(a, as, b, bs, sa, sb, bias, c, M, N, K, scale_vectors, st);
    case 3: return launch_gemm<128, 128, MX, SCALE_KM, OUT, false, I8>(a, as, b, bs, sa, sb, bias, c, M, N, K, scale_vectors, st);
    case 4: return launch_gemm<64, 128, MX, SCALE_KM, OUT, false, I8>(a, as, b, bs, sa, sb, bias, c, M, N, K, scale_vectors, st);
    case 5: return launch_gemm<256, 256, MX, SCALE_KM, OUT, false, I8, true>(a, as, b, bs, sa, sb, bias, c, M, N, K, scale_vectors, st);
    case 6:
      // the int8 MFMA has no 64-deep 32 x 32 form in this pipeline: int8 runs configuration 0 here
      if constexpr (I8) return launch_gemm<256, 256, MX, SCALE_KM, OUT, false, I8>(a, as, b, bs, sa, sb, bias, c, M, N, K, scale_vectors, st);
      else return gemm_w32(MX, SCALE_KM, OUT, a, as, b, bs, sa, sb, bias, c, M, N, K, scale_vectors, st);
    // 192 columns: whole waves of tiles for widths like 12288 at short M (8 x 64 = 512 tiles at
    // M = 2048 where 256-column tiles make 384, one and a half waves)
    case 7: return launch_gemm<256, 192, MX, SCALE_KM, OUT, false, I8>(a, as, b, bs, sa, sb, bias, c, M, N, K, scale_vectors, st);
  }
  return km_fail(KM_ERR_ARG, "km_gemm: unknown config");
}

static int check_gemm_args(const char* who, const void* a, const void* b, void* c, int64_t M, int64_t N,
                           int64_t K, int out_dtype, int config) {
  static thread_local char msg[160];
  if (out_dtype != KM_BF16 && out_dtype != KM_F16) {
    snprintf(msg, sizeof msg, "%s: out_dtype must be bf16 or f16", who);
    return km_fail(KM_ERR_ARG, msg);
  }
  if (M < 0 || N < 0 || K <= 0 || K % kStepBytes) {
    snprintf(msg, sizeof msg, "%s: K=%lld must be a positive multiple of 128", who, (long long)K);
    return km_fail(KM_ERR_UNSUPPORTED, msg);
  }
  if (M * K > 0x7FFFFFFFll || N * K > 0x7FFFFFFFll || M > 0x0FFFFFFF || N > 0x0FFFFFFF) {
    snprintf(msg, sizeof msg, "%s: dimension too large", who);
    return km_fail(KM_ERR_ARG, msg);
  }
  if (config < 0 || config >= kNumGemmConfigs) {
    snprintf(msg, sizeof msg, "%s: config %d out of range", who, config);
    return km_fail(KM_ERR_ARG, msg);
  }
  if (M > 0 && N > 0 && (!a || !b || !c)) {
    snprintf(msg, sizeof msg, "%s: null pointer", who);
    return km_fail(KM_ERR_ARG, msg);
  }
  if ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15) {
    snprintf(msg, sizeof msg, "%s: operands must be 16-byte aligned", who);
    return km_fail(KM_ERR_UNSUPPORTED, msg);
  }
  return KM_OK;
}

int gemm_num_configs() { return kNumGemmConfigs; }
int gemm_config_desc(int config, char* buf, int len) {
  if (config < 0 || config >= kNumGemmConfigs) return km_fail(KM_ERR_ARG, "config out of range");
  const GemmConfig& c = kGemmConfigs[config];
  snprintf(buf, len, "bm=%d,bn=%d,bk=128,waves=4,wg_per_cu=%d,b_stages=%d,mfma=%d", c.bm, c.bn, config == 1 || config == 3 || config == 4 ? 2 : 1, c.b_stages, c.mfma);
  return KM_OK;
}

}  // namespace km

using namespace km;

extern "C" int km_gemm_mx(const void* a, const void* a_scale, const void* b, const void* b_scale,
                          const void* bias, void* c, int64_t M, int64_t N, int64_t K, int out_dtype,
                          int scale_layout, int config, void* stream) {
  int rc = check_gemm_args("km_gemm_mx", a, b, c, M, N, K, out_dtype, config);
  if (rc != KM_OK) return rc;
  if (M == 0 || N == 0) return KM_OK;
  if (!a_scale || !b_scale) return km_fail(KM_ERR_ARG, "km_gemm_mx: null scale pointer");
  if (scale_layout != KM_SCALES_ROWMAJOR && scale_layout != KM_SCALES_PACKED)
    return km_fail(KM_ERR_ARG, "km_gemm_mx: unknown scale layout");
  if ((reinterpret_cast<uintptr_t>(a_scale) | reinterpret_cast<uintptr_t>(b_scale)) & 3)
    return km_fail(KM_ERR_UNSUPPORTED, "km_gemm_mx: scales must be 4-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  const bool km = scale_layout == KM_SCALES_PACKED;
  if (out_dtype == KM_BF16) {
    if (km) return dispatch_config<true, true, KM_BF16>(config, a, a_scale, b, b_scale, nullptr, nullptr, bias, c, (int)M, (int)N, (int)K, 0, st);
    return dispatch_config<true, false, KM_BF16>(config, a, a_scale, b, b_scale, nullptr, nullptr, bias, c, (int)M, (int)N, (int)K, 0, st);
  }
  if (km) return dispatch_config<true, true, KM_F16>(config, a, a_scale, b, b_scale, nullptr, nullptr, bias, c, (int)M, (int)N, (int)K, 0, st);
  return dispatch_config<true, false, KM_F16>(config, a, a_scale, b, b_scale, nullptr, nullptr, bias, c, (int)M, (int)N, (int)K, 0, st);
}

extern "C" int km_gemm_fp8_tensor(const void* a, const float* sa, const void* b, const float* sb,
                                  const void* bias, void* c, int64_t M, int64_t N, int64_t K,
                                  int out_dtype, int config, void* stream) {
  int rc = check_gemm_args("km_gemm_fp8_tensor", a, b, c, M, N, K, out_dtype, config);
  if (rc != KM_OK) return rc;
  if (M == 0 || N == 0) return KM_OK;
  if (!sa || !sb) return km_fail(KM_ERR_ARG, "km_gemm_fp8_tensor: null scale pointer");
  hipStream_t st = (hipStream_t)stream;
  if (out_dtype == KM_BF16)
    return dispatch_config<false, false, KM_BF16>(config, a, nullptr, b, nullptr, sa, sb, bias, c, (int)M, (int)N, (int)K, 0, st);
  return dispatch_config<false, false, KM_F16>(config, a, nullptr, b, nullptr, sa, sb, bias, c, (int)M, (int)N, (int)K, 0, st);
}

extern "C" int km_gemm_fp8_rows(const void* a, const float* sa, const void* b, const float* sb,
                                const void* bias, void* c, int64_t M, int64_t N, int64_t K,
                                int out_dtype, int config, void* stream) {
  int rc = check_gemm_args("km_gemm_fp8_rows", a, b, c, M, N, K, out_dtype, config);
  if (rc != KM_OK) return rc;
  if (M == 0 || N == 0) return KM_OK;
  if (!sa || !sb) return km_fail(KM_ERR_ARG, "km_gemm_fp8_rows: null scale pointer");
  if (reinterpret_cast<uintptr_t>(sb) & 15) return km_fail(KM_ERR_UNSUPPORTED, "km_gemm_fp8_rows: the column scales must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  if (out_dtype == KM_BF16)
    return dispatch_config<false, false, KM_BF16>(config, a, nullptr, b, nullptr, sa, sb, bias, c, (int)M, (int)N, (int)K, 1, st);
  return dispatch_config<false, false, KM_F16>(config, a, nullptr, b, nullptr, sa, sb, bias, c, (int)M, (int)N, (int)K, 1, st);
}

extern "C" int km_gemm_i8_rows(const void* a, const float* sa, const void* b, const float* sb,
                               const void* bias, void* c, int64_t M, int64_t N, int64_t K,
                               int out_dtype, int config, void* stream) {
  int rc = check_gemm_args("km_gemm_i8_rows", a, b, c, M, N, K, out_dtype, config);
  if (rc != KM_OK) return rc;
  if (M == 0 || N == 0) return KM_OK;
  if (!sa) return km_fail(KM_ERR_ARG, "km_gemm_i8_rows: null row scale pointer");
  if (reinterpret_cast<uintptr_t>(sb) & 15) return km_fail(KM_ERR_UNSUPPORTED, "km_gemm_i8_rows: the column scales must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  if (out_dtype == KM_BF16)
    return dispatch_config<false, false, KM_BF16, true>(config, a, nullptr, b, nullptr, sa, sb, bias, c, (int)M, (int)N, (int)K, 1, st);
  return dispatch_config<false, false, KM_F16, true>(config, a, nullptr, b, nullptr, sa, sb, bias, c, (int)M, (int)N, (int)K, 1, st);
}
