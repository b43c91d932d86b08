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
// Shape of the kernel. A workgroup of four wavefronts (2 x 2) owns a BM x 128 tile, so the weight
// scale is one number per workgroup and K step. A wavefront's (BM/2) x 64 sub-tile is walked in
// rows of four MFMA tiles (16 tokens x 64 output columns, which share one activation scale): the
// four MFMAs of a row write a set of partial-sum registers, and between them the partial sums of
// the row before (the other set) are promoted on the vector ALU, so the promotion is issued while
// the matrix pipe is busy. The B fragments of a step stay in registers; A fragments are read a row
// ahead. The operand slabs are fetched STAGES - 1 steps ahead (direct-to-LDS buffer loads into a
// ring of STAGES buffers, the swizzled slab layout of the other fp8 GEMMs); a step waits only for
// the slabs of the step after it, so the fetches of the step after that stay in flight across the
// barrier. The tall tile halves the LDS reads per MFMA of the square one (LDS bandwidth, not the
// matrix pipe, bounds 64 x 64 sub-tiles).
#include <stdio.h>

#include <mutex>

#include "km_gemm_common.h"

namespace km {

constexpr int kBlkTileN = 128;

// Built with -mllvm -amdgpu-mfma-vgpr-form: the MFMAs write ordinary vector registers. Without it
// the compiler puts their results in accumulation registers and copies every partial sum out
// before the promotion (one more vector-ALU instruction per value).
// SA_KMAJOR: the activation scales are laid out [K/128, M] (the quantizer's second output), so
// the tile's scales of a step are one run of BM floats; from the natural [M, K/128] matrix every
// lane of the scale fetch gathers from a row of its own.
// WAVES 8: two wavefronts per SIMD on the same tile (a 4 x 2 grid of (BM/4) x 64 sub-tiles). The loop
// is scheduled by the compiler and its waits (slab and scale fetches, LDS reads, the promotion's
// dependence on the MFMA) stand in the open with one wavefront per SIMD; a second one issues into them.
// BN 256 (with WAVES 8): a 2 x 4 grid of 128 x 64 sub-tiles on a 256 x 256 tile, the operand bytes per
// flop of the MX kernel's large tile; each half of the wavefronts has its own weight-scale block.
template <int OUT, int BM, int STAGES, bool SA_KMAJOR, int WAVES = 4, int BN = kBlkTileN>
__global__ __launch_bounds__(64 * WAVES) void gemm_fp8_blocks_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, const float* __restrict__ sa,
    const float* __restrict__ sb, const uint16_t* __restrict__ bias, uint16_t* __restrict__ C, int M, int N, int K) {
  constexpr int WCOLS = BN / 64;                       // a wavefront's sub-tile is 64 columns wide
  constexpr int NT = 64 * WAVES, WROWS = WAVES / WCOLS;  // wavefronts: WROWS along M x WCOLS along N
  constexpr int TM = BM / (16 * WROWS), TN = 4;        // 16x16 MFMA tiles per wavefront and axis
  static_assert(BN == 128 || (BN == 256 && WAVES == 8), "tile widths");
  constexpr int A_SLAB = BM * kStepBytes, B_SLAB = BN * kStepBytes;
  constexpr int PASS_ROWS = NT / 8, PASS_BYTES = NT * 16;  // 8 lanes per 128-byte row
  constexpr int A_PASSES = BM / PASS_ROWS, B_PASSES = BN / PASS_ROWS;
  static_assert(WAVES == 4 || WAVES == 8, "one or two wavefronts per SIMD");
  constexpr int DMAS = A_PASSES + B_PASSES;     // slab fetch instructions per wavefront and step
  static_assert(STAGES == 2 || STAGES == 3, "ring of two or three slab pairs");
  static_assert(STAGES * (A_SLAB + B_SLAB) <= 160 * 1024, "LDS");
  static_assert(STAGES * A_SLAB >= 2 * 16384 && STAGES * B_SLAB >= 2 * 16384, "epilogue staging: four 16 KiB buffers");
  __shared__ __attribute__((aligned(1024))) uint8_t a_ring[STAGES][A_SLAB];
  __shared__ __attribute__((aligned(1024))) uint8_t b_ring[STAGES][B_SLAB];
  __shared__ __attribute__((aligned(256))) float sa_ring[STAGES][BM];  // the tile's activation scales of a step

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // wavefront index bits: column within a 128-column half, row, (BN 256) which half
  const int wm = (BN == 256 ? (wave >> 1) & 1 : wave >> 1) * (BM / WROWS), wn = (BN == 256 ? (wave >> 2) * 128 : 0) + (wave & 1) * 64;
  const int r16 = lane & 15, g = lane >> 4;
  const int nk = K / kStepBytes;

  // What a tile fixes: its corner, the operand descriptors (rows past the end are fetched as zeros by
  // their range check), the activation-scale descriptor and lane offset, the wavefront's weight-scale row.
  //
  // Activation scales of a step: the tile's BM floats go to LDS with BM / 64 fetches of 4 bytes per lane
  // (one each by the first wavefronts), like the slabs from inline asm: a load the compiler sees would
  // make it wait for every fetch in flight where the value is first used (its count does not include the
  // hidden ones). A lane needs the scales of rows j * 16 + r16 (j < TM) of its wavefront's 16 * TM rows,
  // so the fetch scatters: LDS float i of the ring slot holds row (i / (16 TM)) * 16 TM + (i % TM) * 16 +
  // (i / TM) % 16, and a lane reads its TM scales as one or two 16-byte LDS reads. (One 4-byte global load
  // per scale and lane, TM a step and wavefront, held the matrix pipe up for a sixth of the kernel's time.)
  // Natural layout: the descriptor starts at the tile's first row, so rows past M read as zero scales
  // (their partial sums are zeros as well). K-major: a row past M reads a neighbour's scale or, past the
  // end, zero; its sums are never stored.
  struct Tile {
    int m0, n0, sa_voff;
    v4i a_rsrc, b_rsrc, sa_rsrc;
    const float* sb_row;
  };
  constexpr int SA_FETCHES = BM / 64;  // wavefront w < SA_FETCHES fetches LDS floats [64 w, 64 w + 64) of a slot
  static_assert(SA_FETCHES <= WAVES, "one scale fetch per wavefront at most");
  const int sa_slot_index = (wave * 64 + lane) % BM;
  const int sa_row = sa_slot_index / (16 * TM) * (16 * TM) + (sa_slot_index % TM) * 16 + (sa_slot_index / TM) % 16;
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  auto tile_at = [&](int pid) __attribute__((always_inline)) -> Tile {
    int tile_m, tile_n;
    tile_of(pid, tiles_m, tiles_n, tile_m, tile_n);
    Tile t;
    t.m0 = tile_m * BM;
    t.n0 = tile_n * BN;
    t.a_rsrc = raw_rsrc(A + (size_t)t.m0 * K, (uint32_t)min((int64_t)(M - t.m0) * K, (int64_t)0x7FFFFFFF));
    t.b_rsrc = raw_rsrc(B + (size_t)t.n0 * K, (uint32_t)min((int64_t)(N - t.n0) * K, (int64_t)0x7FFFFFFF));
    t.sa_rsrc = SA_KMAJOR ? raw_rsrc(sa, (uint32_t)min((int64_t)M * nk * 4, (int64_t)0x7FFFFFFF))
                          : raw_rsrc(sa + (size_t)t.m0 * nk, (uint32_t)min((int64_t)(M - t.m0) * nk * 4, (int64_t)0x7FFFFFFF));
    t.sa_voff = SA_KMAJOR ? (t.m0 + sa_row) * 4 : sa_row * nk * 4;
    t.sb_row = sb + (size_t)min((t.n0 + wn) >> 7, (N - 1) >> 7) * nk;  // the wavefront's 128-column weight block
    return t;
  };
  // PERSIST: a work-group walks tiles pid, pid + grid, ... and fetches the first slabs and scales of
  // the tile after this one during this tile's last K step, so only the epilogue stands between the
  // MFMAs of two tiles. The epilogue stages in the slot the last step read, the early slabs land in the
  // other one, which the walk takes for slot 0 again: the host launches fewer work-groups than tiles
  // only when the number of K steps is even.
  constexpr bool PERSIST = WAVES == 8 && STAGES == 2;
  int pid = blockIdx.x;
  Tile T = tile_at(pid);
  // staging map of a pass: 8 lanes per row; 16 lanes cover rows r and r+8 (one LDS line)
  const int w = tid >> 3;
  const int srow = ((w >> 4) << 4) + ((w & 1) << 3) + ((w >> 1) & 7);
  const int src_chunk = (tid & 7) ^ (srow & 7);
  const int ld_voff = srow * K + src_chunk * 16;
  const int pass_stride = PASS_ROWS * K;
  // fetch p of a step's DMAS: the B passes, then the A passes
  auto dma_pass = [&](const Tile& t, uint8_t* abuf, uint8_t* bbuf, int koff, int p) __attribute__((always_inline)) {
    if (p < B_PASSES) hidden_dma_b128(t.b_rsrc, lds_offset(bbuf) + p * PASS_BYTES + wave * 1024, ld_voff + p * pass_stride, koff);
    else hidden_dma_b128(t.a_rsrc, lds_offset(abuf) + (p - B_PASSES) * PASS_BYTES + wave * 1024, ld_voff + (p - B_PASSES) * pass_stride, koff);
  };
  auto dma = [&](const Tile& t, uint8_t* abuf, uint8_t* bbuf, int ks) __attribute__((always_inline)) {
    const int koff = __builtin_amdgcn_readfirstlane(ks * kStepBytes);
#pragma unroll
    for (int p = 0; p < DMAS; ++p) dma_pass(t, abuf, bbuf, koff, p);
  };
  auto fragment = [&](const uint8_t* slab, int row) __attribute__((always_inline)) -> v8i {
    const v4i lo = *reinterpret_cast<const v4i*>(slab + slab_offset(row, g));
    const v4i hi = *reinterpret_cast<const v4i*>(slab + slab_offset(row, g + 4));
    return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };

  // the activation scales of step ks of tile t, into ring slot `slot`
  auto sa_fetch = [&](const Tile& t, int ks, int slot) __attribute__((always_inline)) {
    if (wave < SA_FETCHES)
      hidden_touch_b32(t.sa_rsrc, lds_offset(&sa_ring[slot][0]) + wave * 256, t.sa_voff, __builtin_amdgcn_readfirstlane(SA_KMAJOR ? ks * M * 4 : ks * 4));
  };
  const int sa_lane = wm + r16 * TM;  // first of this lane's TM floats in a slot

  // weight scale of the step ahead: fetched a step early
  float sb_next = T.sb_row[0];
  // prologue: the scales of step 0 and the slabs of the first STAGES - 1 steps; wait for step 0 only
  sa_fetch(T, 0, 0);
  dma(T, a_ring[0], b_ring[0], 0);
  if (STAGES == 3 && nk > 1) {
    dma(T, a_ring[1], b_ring[1], 1);
    __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(DMAS));
  } else {
    __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));
  }
  __syncthreads();
  __builtin_amdgcn_sched_barrier(0);

  const int total = tiles_m * tiles_n;
  for (;;) {
    const int pid_after = pid + (int)gridDim.x;
    const bool more = PERSIST && pid_after < total;
    const Tile U = tile_at(more ? pid_after : pid);  // the tile after this one

    v4f acc[TN][TM];
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
      for (int j = 0; j < TM; ++j) acc[t][j] = v4f{0.f, 0.f, 0.f, 0.f};

    // One K step: the slabs of step ks are in ring slot `cur`; slot `pre` (read last in the step
    // before, behind that step's barrier) takes the slabs of step ks + STAGES - 1 or, in the last step
    // of a tile that has a successor, the successor's first.
    auto step = [&](int ks, auto cur_tag, auto pre_tag) __attribute__((always_inline)) {
      constexpr int cur = decltype(cur_tag)::value, pre = decltype(pre_tag)::value;
      const uint8_t* a_cur = a_ring[cur];
      const uint8_t* b_cur = b_ring[cur];
      constexpr int nxt = (cur + 1) % STAGES;  // ring slot of step ks + 1
      float s_cur[TM];
#pragma unroll
      for (int j4 = 0; j4 < TM; j4 += 4) {
        const v4f four = *reinterpret_cast<const v4f*>(&sa_ring[cur][sa_lane + j4]);
#pragma unroll
        for (int j = 0; j < 4; ++j) s_cur[j4 + j] = four[j] * sb_next;
      }
      const bool ahead = ks + STAGES - 1 < nk;
      // what this step fetches: the scales of the step after it and the slabs STAGES - 1 steps on, or (the
      // last step of a tile that has a successor) the successor's first scales and slabs
      const bool wraps = more && ks == nk - 1;
      const Tile& from = wraps ? U : T;
      const int ks_scales = wraps ? 0 : min(ks + 1, nk - 1);
      sb_next = from.sb_row[ks_scales];
      sa_fetch(from, ks_scales, nxt);
      const bool fetch = ahead || wraps;
      const int koff = __builtin_amdgcn_readfirstlane((wraps ? 0 : ks + STAGES - 1) * kStepBytes);
      // The slab fetches of the 256-row tiles go behind the MFMAs of the first row of tiles, half of them
      // ahead of the second row and half ahead of the third: at the top of the step, where every wavefront
      // would queue its fetches at the one address unit, nothing else runs meanwhile (2 % on the large
      // tile). The 128-row tile, two work-groups per compute unit, is 3 % faster with them at the top.
      constexpr int kFetchRow = BM >= 256 ? 1 : 0, kFetchRows = BM >= 256 ? 2 : 1;
      static_assert(kFetchRow + kFetchRows <= TM, "fetch rows");
      v8i wf[TN];
#pragma unroll
      for (int t = 0; t < TN; ++t) wf[t] = fragment(b_cur, wn + t * 16 + r16);
      v8i xf = fragment(a_cur, wm + r16);
      v4f part[2][TN];
      static_for<TM + 1>([&](auto j_tag) __attribute__((always_inline)) {
        constexpr int j = decltype(j_tag)::value;
        v8i xf_next = xf;
        if constexpr (j >= kFetchRow && j < kFetchRow + kFetchRows) {
          if (fetch) {
            constexpr int per = (DMAS + kFetchRows - 1) / kFetchRows;
#pragma unroll
            for (int p = (j - kFetchRow) * per; p < (j - kFetchRow + 1) * per && p < DMAS; ++p) dma_pass(from, a_ring[pre], b_ring[pre], koff, p);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (j + 1 < TM) xf_next = fragment(a_cur, wm + (j + 1) * 16 + r16);
        static_for<TN>([&](auto t_tag) __attribute__((always_inline)) {
          constexpr int t = decltype(t_tag)::value;
          // MFMA rows come from B (output columns n), MFMA columns from A (tokens m); unit scales
          if constexpr (j < TM)
            part[j & 1][t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[t], xf, v4f{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
          if constexpr (j > 0) {
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[t][j - 1][v] = __builtin_fmaf(part[(j - 1) & 1][t][v], s_cur[j - 1], acc[t][j - 1][v]);
            // pins the promotion ahead of the wait below (the compiler would sink it past the barrier)
            asm volatile("" : "+v"(acc[t][j - 1]));
          }
          __builtin_amdgcn_sched_barrier(0);
        });
        xf = xf_next;
      });
      // The slabs and scales of step ks + 1 must have landed (STAGES 3: the DMAS newest fetches, those
      // of step ks + 2, stay in flight: vector-memory results return in order) and this step's LDS reads
      // must be done before the barrier lets another wavefront overwrite the slot.
      if (STAGES == 3 && ahead) __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(DMAS));
      else __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));
      __syncthreads();
      __builtin_amdgcn_sched_barrier(0);
    };
    using i0 = std::integral_constant<int, 0>;
    using i1 = std::integral_constant<int, 1>;
    using i2 = std::integral_constant<int, 2>;
    if constexpr (STAGES == 2) {
      for (int ks = 0; ks < nk; ks += 2) {
        step(ks, i0{}, i1{});
        if (ks + 1 < nk) step(ks + 1, i1{}, i0{});
      }
    } else {
      for (int ks = 0; ks < nk; ks += 3) {
        step(ks, i0{}, i2{});
        if (ks + 1 < nk) step(ks + 1, i1{}, i0{});
        if (ks + 2 < nk) step(ks + 2, i2{}, i1{});
      }
    }

    // Every fetch has landed and every wavefront is past its last LDS read. The slot of the last step
    // is free for staging (with a successor, the other slot holds its first slabs).
    const int last_slot = (nk - 1) % STAGES;
    uint8_t* ea = &a_ring[0][0] + last_slot * A_SLAB;
    uint8_t* eb = &b_ring[0][0] + last_slot * B_SLAB;
    if constexpr (WAVES == 4) {
      // four 16 KiB buffers: with the square tile they are the whole ring
      ea = &a_ring[0][0];
      eb = &b_ring[0][0];
      store_tile<BM, BN, OUT, 0, false, false>(acc, 1.0f, nullptr, nullptr, bias, C, M, N, T.m0, T.n0, ea, ea + 16384, eb, eb + 16384);
    } else if constexpr (BN == 128) {
      // each group of four wavefronts writes its half of the tile's rows, staging in a ring of its own
      uint8_t* stage = wave < 4 ? ea : eb;
      store_tile<BM / 2, BN, OUT, 0, false, false>(acc, 1.0f, nullptr, nullptr, bias, C, M, N, T.m0 + (wave >> 2) * (BM / 2), T.n0, stage, stage + 4096,
                                                   stage + 8192, stage + 12288);
    } else {
      // each group of four wavefronts writes its 128-column half of the tile
      uint8_t* stage = wave < 4 ? ea : eb;
      store_tile<BM, 128, OUT, 0, false, false>(acc, 1.0f, nullptr, nullptr, bias, C, M, N, T.m0, T.n0 + (wave >> 2) * 128, stage, stage + 4096,
                                                stage + 8192, stage + 12288);
    }
    if (!more) break;
    // the staging reads are done before the successor's step 0 fetches into this slot
    __syncthreads();
    pid = pid_after;
    T = U;
  }
}

struct BlocksConfig {
  int bm, stages, waves, bn;
};
// the tall tile first (fewest operand and LDS bytes per flop); the square one for short M and small grids;
// the tall tile with two wavefronts per SIMD
static const BlocksConfig kBlocksConfigs[] = {{256, 3, 4, 128}, {128, 2, 4, 128}, {256, 3, 8, 128}, {256, 2, 8, 256}};
constexpr int kNumBlocksConfigs = 4;

int blocks_gemm_num_configs() { return kNumBlocksConfigs; }
int blocks_gemm_config_desc(int config, char* buf, int len) {
  if (config < 0 || config >= kNumBlocksConfigs) return km_fail(KM_ERR_ARG, "config out of range");
  const BlocksConfig& c = kBlocksConfigs[config];
  snprintf(buf, len, "bm=%d,bn=%d,bk=128,waves=%d,stages=%d,wg_per_cu=%d", c.bm, c.bn, c.waves, c.stages, c.bm == 256 ? 1 : 2);
  return KM_OK;
}

// compute units of the current device, asked once per device
static int compute_units() {
  static std::mutex mu;
  static int seen[64];
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 0;
  std::lock_guard<std::mutex> lock(mu);
  if (seen[device] == 0) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) return 0;
    seen[device] = cus;
  }
  return seen[device];
}

template <int OUT, int BM, int STAGES, int WAVES = 4, int BN = kBlkTileN>
static void launch_blocks(const void* a, const float* sa, const void* b, const float* sb, const void* bias, void* c,
                          int M, int N, int K, bool sa_kmajor, hipStream_t st) {
  const int tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  // The kernel that walks tiles (two stages, eight wavefronts) holds one work-group per compute unit:
  // launch one per unit, a multiple of the 8 XCDs so that tile pid + grid stays on the XCD of tile pid.
  // An odd number of K steps would leave the early slabs in the wrong ring slot: one work-group per tile then.
  int grid = tiles;
  if (WAVES == 8 && STAGES == 2 && (K / kStepBytes) % 2 == 0) {
    const int units = compute_units();
    if (units >= kXcds && units - units % kXcds < tiles) grid = units - units % kXcds;
  }
  if (sa_kmajor)
    hipLaunchKernelGGL((gemm_fp8_blocks_kernel<OUT, BM, STAGES, true, WAVES, BN>), dim3(grid), dim3(64 * WAVES), 0, st, (const uint8_t*)a,
                       (const uint8_t*)b, sa, sb, (const uint16_t*)bias, (uint16_t*)c, M, N, K);
  else
    hipLaunchKernelGGL((gemm_fp8_blocks_kernel<OUT, BM, STAGES, false, WAVES, BN>), dim3(grid), dim3(64 * WAVES), 0, st, (const uint8_t*)a,
                       (const uint8_t*)b, sa, sb, (const uint16_t*)bias, (uint16_t*)c, M, N, K);
}

}  // namespace km

using namespace km;

extern "C" int km_gemm_fp8_blocks(const void* a, const float* sa, const void* b, const float* sb,
                                  const void* bias, void* c, int64_t M, int64_t N, int64_t K,
                                  int out_dtype, int sa_layout, int config, void* stream) {
  if (out_dtype != KM_BF16 && out_dtype != KM_F16) return km_fail(KM_ERR_ARG, "km_gemm_fp8_blocks: out_dtype must be bf16 or f16");
  if (M < 0 || N < 0 || K <= 0 || K % kStepBytes) return km_fail(KM_ERR_UNSUPPORTED, "km_gemm_fp8_blocks: K must be a positive multiple of 128");
  if (M * K > 0x7FFFFFFFll || N * K > 0x7FFFFFFFll || M > 0x0FFFFFFF || N > 0x0FFFFFFF)
    return km_fail(KM_ERR_ARG, "km_gemm_fp8_blocks: dimension too large");
  if (config < 0 || config >= kNumBlocksConfigs) return km_fail(KM_ERR_ARG, "km_gemm_fp8_blocks: config out of range");
  if (sa_layout != KM_SCALES_ROWMAJOR && sa_layout != KM_SCALES_KMAJOR) return km_fail(KM_ERR_ARG, "km_gemm_fp8_blocks: unknown activation scale layout");
  if (M == 0 || N == 0) return KM_OK;
  if (!a || !b || !c || !sa || !sb) return km_fail(KM_ERR_ARG, "km_gemm_fp8_blocks: null pointer");
  if ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15)
    return km_fail(KM_ERR_UNSUPPORTED, "km_gemm_fp8_blocks: operands must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  const bool km = sa_layout == KM_SCALES_KMAJOR;
  if (out_dtype == KM_BF16) {
    if (config == 0) launch_blocks<KM_BF16, 256, 3>(a, sa, b, sb, bias, c, (int)M, (int)N, (int)K, km, st);
    else if (config == 1) launch_blocks<KM_BF16, 128, 2>(a, sa, b, sb, bias, c, (int)M, (int)N, (int)K, km, st);
    else if (config == 2) launch_blocks<KM_BF16, 256, 3, 8>(a, sa, b, sb, bias, c, (int)M, (int)N, (int)K, km, st);
    else launch_blocks<KM_BF16, 256, 2, 8, 256>(a, sa, b, sb, bias, c, (int)M, (int)N, (int)K, km, st);
  } else {
    if (config == 0) launch_blocks<KM_F16, 256, 3>(a, sa, b, sb, bias, c, (int)M, (int)N, (int)K, km, st);
    else if (config == 1) launch_blocks<KM_F16, 128, 2>(a, sa, b, sb, bias, c, (int)M, (int)N, (int)K, km, st);
    else if (config == 2) launch_blocks<KM_F16, 256, 3, 8>(a, sa, b, sb, bias, c, (int)M, (int)N, (int)K, km, st);
    else launch_blocks<KM_F16, 256, 2, 8, 256>(a, sa, b, sb, bias, c, (int)M, (int)N, (int)K, km, st);
  }
  return km_check_launch("km_gemm_fp8_blocks");
}
