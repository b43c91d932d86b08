// Machinery shared by the GEMM kernels: the swizzled LDS slab layout, the work-group to tile
// map, 16-bit packing, compile-time loops and the epilogue that writes a wavefront's
// accumulators through an LDS transpose.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>
#include <utility>

#include "km_internal.h"
#include "km_numeric.h"
#include "km_tile_plan.h"

namespace km {


typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kStepBytes = 128;  // K bytes per step (= K elements, e4m3)

__device__ __forceinline__ int slab_offset(int row, int chunk) {
  return (((row >> 4) * 8 + (row & 7)) << 8) + (((row >> 3) & 1) << 7) + ((chunk ^ (row & 7)) << 4);
}

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// two fp32 -> two 16-bit values in one register, round to nearest even (one v_cvt_pk_* each)
template <int OUT>
__device__ __forceinline__ uint32_t pack2(float a, float b);
template <>
__device__ __forceinline__ uint32_t pack2<KM_BF16>(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{a, b}), bf16x2));
}
template <>
__device__ __forceinline__ uint32_t pack2<KM_F16>(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{a, b}), f16x2));
}
template <int OUT>
__device__ __forceinline__ float unpack1(uint32_t h);
template <>
__device__ __forceinline__ float unpack1<KM_BF16>(uint32_t h) { return bits_f32(h << 16); }
template <>
__device__ __forceinline__ float unpack1<KM_F16>(uint32_t h) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

// compile-time loop: f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>)
template <class F, int... Is>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, Is...>) {
  (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

typedef __attribute__((address_space(3))) void* lds_ptr_t;

// s_waitcnt immediates (gfx9 encoding: vmcnt [3:0]+[15:14], expcnt [6:4], lgkmcnt [11:8])
constexpr int kWaitVm0 = 0x0F70;         // vmcnt(0)
constexpr int kWaitLgkm0 = 0xC07F;       // lgkmcnt(0)
constexpr int wait_vm_lgkm0(int n) { return (n & 15) | ((n >> 4) << 14) | 0x0070; }  // vmcnt(n) lgkmcnt(0)

// ---- vector-memory reads the compiler does not see ------------------------------------------
// The compiler cannot tell which LDS buffer a direct-to-LDS load fills and answers every later
// LDS read with s_waitcnt vmcnt(0), which drains the prefetches that are meant to stay in
// flight across a K step. Issued from inline asm, the loads are invisible to that bookkeeping:
// the only vmcnt waits left are the explicit ones of the kernel, and every result is used after
// one of them (a "memory" clobber keeps LDS reads from moving across). The hazard recognizer
// does not look into inline asm either: an SGPR written by a VALU instruction (v_readfirstlane,
// the reload of a spilled SGPR) must not be read by a vector-memory instruction within 5 wait
// states, and m0 not within 1, hence the s_nop in front of each. The direct-to-LDS load takes its
// LDS address from m0, which the statement writes itself and declares as clobbered.
__device__ __forceinline__ uint32_t lds_offset(const void* p) {
  return (uint32_t)reinterpret_cast<uintptr_t>((lds_ptr_t)const_cast<void*>(p));
}
// raw buffer descriptor (stride 0, range check on the per-lane offset) from uniform values
__device__ __forceinline__ v4i raw_rsrc(const void* base, uint32_t bytes) {
  const uint64_t b = (uint64_t)reinterpret_cast<uintptr_t>(base);
  return v4i{__builtin_amdgcn_readfirstlane((int)(uint32_t)b), __builtin_amdgcn_readfirstlane((int)((uint32_t)(b >> 32) & 0xFFFFu)),
             __builtin_amdgcn_readfirstlane((int)bytes), 0x00020000};
}
// each lane fetches 16 bytes at voffset (+ soffset); they land at lds_addr + 16 * lane
// (the compiler keeps m0 out of its own allocation and says so when it sees it in a clobber list)
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void hidden_dma_b128(const v4i& rsrc, uint32_t lds_addr, int voffset, int soffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               ::"s"(lds_addr), "v"(voffset), "s"(rsrc), "s"(soffset) : "memory", "m0");
}
// The same load for use inside a K loop whose SGPR operands (descriptor, soffset, the LDS address) are
// loop invariant or written by the scalar ALU: only m0 needs its one wait state. The five wait states of
// the general form keep the matrix pipe idle once per load when it rides behind an MFMA.
__device__ __forceinline__ void loop_dma_b128(const v4i& rsrc, uint32_t lds_addr, int voffset, int soffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               ::"s"(lds_addr), "v"(voffset), "s"(rsrc), "s"(soffset) : "memory", "m0");
}
// 4 bytes per lane to lds_addr + 4 * lane: used to pull lines into L2 ahead of their real fetch,
// aimed at LDS bytes that a later load of the same wavefront overwrites
__device__ __forceinline__ void hidden_touch_b32(const v4i& rsrc, uint32_t lds_addr, int voffset, int soffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\tbuffer_load_dword %1, %2, %3 offen lds"
               ::"s"(lds_addr), "v"(voffset), "s"(rsrc), "s"(soffset) : "memory", "m0");
}
#pragma clang diagnostic pop
__device__ __forceinline__ uint64_t hidden_load_b64(const v4i& rsrc, int voffset, int soffset) {
  uint64_t v;
  asm volatile("s_nop 4\n\tbuffer_load_dwordx2 %0, %1, %2, %3 offen" : "=v"(v) : "v"(voffset), "s"(rsrc), "s"(soffset) : "memory");
  return v;
}
__device__ __forceinline__ uint32_t hidden_load_b32(const v4i& rsrc, int voffset, int soffset) {
  uint32_t v;
  asm volatile("s_nop 4\n\tbuffer_load_dword %0, %1, %2, %3 offen" : "=v"(v) : "v"(voffset), "s"(rsrc), "s"(soffset) : "memory");
  return v;
}

__device__ __forceinline__ int fresh_thread_index() {
  int tid = threadIdx.x;
  asm volatile("" : "+v"(tid));
  return tid;
}

// The interior-tile path of the epilogues: a wavefront writes its WTM x WTN sub-tile of 16-bit
// values, 16 rows (one row of MFMA tiles) per pass, through an LDS region of its own of 16 rows
// of WTN * 2 + 16 bytes. `item(j, t)` yields the 8 bytes of this lane for piece t (0 .. NT-1) of
// pass j and `col_byte(t)` where they go in the lane's row r16 of the region (negative: the lane
// has no such piece); the region is read
// back along rows, 16 bytes a lane, and stored as whole WTN*2-byte row segments (full 128-byte
// lines) with 16-byte streaming stores (the output is not read again by the kernel and should
// not push the operand slabs out of L2; plain stores issue twice as fast and make the K loop
// 15 % slower).
//
// One wavefront per SIMD has nothing else to run while it waits, so the passes are pipelined by
// hand: the transposed rows of pass j are on their way from LDS to registers, and then to memory
// one store at a time, between the pieces of pass j + 1 as these are read out of the
// accumulators, rounded and written to LDS. LDS operations of a wavefront execute in order, so
// pass j + 1 may overwrite the region right behind the reads of pass j. The scheduling barriers
// keep this order: left alone, the compiler copies all accumulators out first and then has one
// set of registers for every row, with a full LDS round trip per store.
template <int WTN, int TM, int NT, class Item, class ColByte>
__device__ __forceinline__ void staged_rows_out(uint8_t* region, uint8_t* out_base, int N, int lane, Item&& item, ColByte&& col_byte) {
  constexpr int RP = WTN * 2 + 16;   // LDS row pitch in bytes: the 64 lanes of a write spread evenly over the banks
  constexpr int LPR = WTN * 2 / 16;  // 16-byte pieces per row on the read side
  constexpr int NRD = 16 * LPR / 64; // reads (and stores) per pass: the pass's 16 LPR pieces, 64 per instruction
  static_assert((16 * LPR) % 64 == 0 && NT >= NRD, "whole instructions per pass, at least a piece between two stores");
  const int r16 = lane & 15;
  // piece 64 i + lane of a pass is (row, 16-byte column) = (piece / LPR, piece % LPR): its LDS offset
  // and its offset from the pass's first output row, 32 bits (row < 16): a uniform row pointer per
  // pass and no 64-bit vector arithmetic per store
  uint32_t lds_off[NRD], out_off[NRD];
#pragma unroll
  for (int i = 0; i < NRD; ++i) {
    const int piece = i * 64 + lane;
    lds_off[i] = (uint32_t)((piece / LPR) * RP + (piece % LPR) * 16);
    out_off[i] = (uint32_t)(piece / LPR) * (uint32_t)N * 2u + (uint32_t)(piece % LPR) * 16u;
  }
  v4i rd[NRD];
  auto store_one = [&](int pass, int i) __attribute__((always_inline)) {
    uint8_t* rows = out_base + (size_t)(pass * 16) * N * 2;
    __builtin_nontemporal_store(rd[i], reinterpret_cast<v4i*>(rows + out_off[i]));
  };
  static_for<TM>([&](auto j_tag) __attribute__((always_inline)) {
    constexpr int j = decltype(j_tag)::value;
    static_for<NT>([&](auto t_tag) __attribute__((always_inline)) {
      constexpr int t = decltype(t_tag)::value;
      const uint2 piece = item(j_tag, t_tag);
      const int at = col_byte(t);  // negative: this lane has no piece t
      if (at >= 0) *reinterpret_cast<uint2*>(region + r16 * RP + at) = piece;
      // store i of the pass before goes behind piece (i + 1) NT / NRD - 1
      if constexpr (j > 0 && ((t + 1) * NRD) / NT > (t * NRD) / NT) store_one(j - 1, (t * NRD) / NT);
      __builtin_amdgcn_sched_barrier(0);
    });
#pragma unroll
    for (int i = 0; i < NRD; ++i) rd[i] = *reinterpret_cast<const v4i*>(region + lds_off[i]);
    __builtin_amdgcn_sched_barrier(0);
  });
#pragma unroll
  for (int i = 0; i < NRD; ++i) store_one(TM - 1, i);
}
constexpr int staged_rows_bytes(int wtn) { return 16 * (wtn * 2 + 16); }

// Epilogue of a 2 x 2 wavefront grid over a BM x BN tile of 16x16 MFMA tiles whose rows are
// output columns: lane (r16 = lane%16, g = lane/16) of tile (t, j) holds
// C[m0+wm+j*16+r16][n0+wn+t*16+4g .. +3]. Computes acc * post * row_scale[m] * col_scale[n] +
// bias[n] in fp32 (either scale vector may be null), rounds once to the 16-bit output type. `bufs` are four LDS buffers of at least
// `buf_bytes` each, free for staging (one per wavefront).
// SCALED 0: acc + bias; 1: acc * (row * col scale) + bias, fused; 2: the accumulator holds int32
// bits: ((float(acc) * row scale) * col scale) + bias with every product and the sum rounded
// on its own, the order of the reference's int8 linear (src/kohakumoss_kernels/int8/op.py:45-48).
// A workgroup of eight wavefronts calls it once per group of four (wavefront index modulo 4,
// m0 of that group's rows) with SYNC off, after a barrier of its own: the groups may take
// different branches here.
// ACC_AGPR: the accumulators live in AGPRs (kernels whose MFMAs are opaque statements with tied
// "a" operands). Each element is then copied to a vector register by a statement of its own right
// where it is consumed, inside its pass; left to the compiler, the 256 copies sit behind the K
// loop, where they leave no register for anything else.
template <bool ACC_AGPR>
__device__ __forceinline__ float acc_element(const v4f& a, int v) {
  if constexpr (ACC_AGPR) {
    float r;
    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(r) : "a"(a[v]));
    return r;
  } else {
    return a[v];
  }
}
// CLEAR: every accumulator is set to zero once it has been read (a work-group that goes on to
// another tile starts its K loop without a pass over the 256 registers).
template <int BM, int BN, int OUT, int SCALED, bool SYNC = true, bool ACC_AGPR = true, bool CLEAR = false>
__device__ __forceinline__ void store_tile(v4f (&acc)[BN / 32][BM / 32], float post, const float* __restrict__ row_scale,
                                           const float* __restrict__ col_scale, const uint16_t* __restrict__ bias, uint16_t* __restrict__ C, int M, int N,
                                           int m0, int n0, uint8_t* buf0, uint8_t* buf1, uint8_t* buf2, uint8_t* buf3) {
  constexpr int WTM = BM / 2, WTN = BN / 2, TM = WTM / 16, TN = WTN / 16;
  // The thread index is taken afresh and made opaque: lane-derived values of the main loop must
  // not stay live into the epilogue, where every accumulator is read out and registers run short
  // (a value that is spilled here would be reloaded at each of its uses inside the loop).
  const int tid = fresh_thread_index();
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6) & 3;
  const int wm = (wave >> 1) * WTM, wn = (wave & 1) * WTN;
  const int r16 = lane & 15, g = lane >> 4;
  const bool has_bias = bias != nullptr;
  auto value = [&](float a, float rs, float cs, float b) __attribute__((always_inline)) {
    if constexpr (SCALED == 2) {
#pragma clang fp contract(off)  // three roundings: a fused multiply-add would differ where the sum cancels
      const float scaled_rows = (float)__builtin_bit_cast(int, a) * rs;
      const float scaled = scaled_rows * cs;
      return scaled + b;
    } else if constexpr (SCALED == 1) return a * (rs * cs) + b;
    else return a + b;
  };
  if (m0 + BM <= M && n0 + BN <= N && (N & 7) == 0) {
    // Interior tile. A lane holds 4 consecutive n of 16 different rows per MFMA tile; storing
    // that directly makes 32-byte write requests. Each wavefront transposes its sub-tile through
    // LDS (idle now) instead.
    // (each of the four buffers holds staged_rows_bytes(WTN) bytes)
    if constexpr (SYNC) __syncthreads();  // every wavefront is done reading fragments
    uint8_t* region = wave == 0 ? buf0 : wave == 1 ? buf1 : wave == 2 ? buf2 : buf3;
    uint8_t* out_base = reinterpret_cast<uint8_t*>(C) + ((size_t)(m0 + wm) * N + n0 + wn) * 2;  // uniform
    auto all_passes = [&](auto bias_tag) __attribute__((always_inline)) {
      constexpr bool ADD = decltype(bias_tag)::value;
      float bv[TN][4], cs[TN][4], rs[TM];
      if constexpr (ADD) {
        uint2 braw[TN];
#pragma unroll
        for (int t = 0; t < TN; ++t) braw[t] = make_uint2(0u, 0u);
        if (has_bias) {
          const uint16_t* bias_lane = bias + n0 + wn + 4 * g;
#pragma unroll
          for (int t = 0; t < TN; ++t) braw[t] = *reinterpret_cast<const uint2*>(bias_lane + t * 16);
        }
#pragma unroll
        for (int t = 0; t < TN; ++t) {
          bv[t][0] = unpack1<OUT>(braw[t].x & 0xFFFFu); bv[t][1] = unpack1<OUT>(braw[t].x >> 16);
          bv[t][2] = unpack1<OUT>(braw[t].y & 0xFFFFu); bv[t][3] = unpack1<OUT>(braw[t].y >> 16);
          cs[t][0] = cs[t][1] = cs[t][2] = cs[t][3] = 1.f;
          if constexpr (SCALED != 0) {
            if (col_scale != nullptr) {
              const float4 c4 = *reinterpret_cast<const float4*>(col_scale + n0 + wn + 4 * g + t * 16);
              cs[t][0] = c4.x; cs[t][1] = c4.y; cs[t][2] = c4.z; cs[t][3] = c4.w;
            }
          }
        }
#pragma unroll
        for (int j = 0; j < TM; ++j) rs[j] = (SCALED != 0 && row_scale != nullptr) ? post * row_scale[m0 + wm + j * 16 + r16] : post;
      }
      staged_rows_out<WTN, TM, TN>(
          region, out_base, N, lane,
          [&](auto j_tag, auto t_tag) __attribute__((always_inline)) {
            constexpr int j = decltype(j_tag)::value, t = decltype(t_tag)::value;
            float o[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
              const float a = acc_element<ACC_AGPR>(acc[t][j], v);
              if constexpr (SCALED == 0 && !ADD) o[v] = a;
              else o[v] = value(a, rs[j], cs[t][v], bv[t][v]);
            }
            if constexpr (CLEAR) {
              acc[t][j] = v4f{0.f, 0.f, 0.f, 0.f};
              asm volatile("" : "+a"(acc[t][j]));
            }
            return make_uint2(pack2<OUT>(o[0], o[1]), pack2<OUT>(o[2], o[3]));
          },
          [&](int t) __attribute__((always_inline)) { return (t * 16 + 4 * g) * 2; });
    };
    // without a bias and without scales the accumulator is rounded as it is
    if (SCALED != 0 || has_bias) all_passes(std::true_type{});
    else all_passes(std::false_type{});
    return;
  }
  const bool vec_ok = (N & 3) == 0;
#pragma unroll
  for (int t = 0; t < TN; ++t) {
    const int n = n0 + wn + t * 16 + 4 * g;
    float bv[4] = {0.f, 0.f, 0.f, 0.f}, cs[4] = {1.f, 1.f, 1.f, 1.f};
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      if (has_bias && n + v < N) bv[v] = unpack1<OUT>(bias[n + v]);
      if (col_scale != nullptr && n + v < N) cs[v] = col_scale[n + v];
    }
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      const int m = m0 + wm + j * 16 + r16;
      if (m >= M || n >= N) continue;
      const float rs = row_scale != nullptr ? post * row_scale[m] : post;
      float o[4];
#pragma unroll
      for (int v = 0; v < 4; ++v) o[v] = value(acc_element<ACC_AGPR>(acc[t][j], v), rs, cs[v], bv[v]);
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
  if constexpr (CLEAR) {
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
      for (int j = 0; j < TM; ++j) {
        acc[t][j] = v4f{0.f, 0.f, 0.f, 0.f};
        asm volatile("" : "+a"(acc[t][j]));
      }
  }
}

}  // namespace km
