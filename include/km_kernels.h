/* C ABI of the MI355X (gfx950) quantized-linear kernels.
 *
 * The reference (KohakuMossTrainer, pure Python) has no FFI of its own: its backends are
 * Python modules that register a launcher pair per op
 *     register_launchers(backend, fwd, dgrad)      src/kohakumoss_kernels/fp8/op.py:43-46
 *                                                  src/kohakumoss_kernels/quant/__init__.py:66-68
 * and the Triton backend's launchers call JIT kernels. This library is what a "hip"
 * backend's launchers call instead, through ctypes. Every entry point
 *   - takes plain device pointers, sizes and a hipStream_t (as void*; NULL = the null stream),
 *   - launches asynchronously on that stream, never synchronizes, never allocates,
 *   - never writes its inputs,
 *   - returns KM_OK or a negative error code; km_last_error() then describes it
 *     (thread local). The Python side turns a non-zero code into RuntimeError, the
 *     reference's "cannot build / launch here" class (src/kohakumoss_kernels/errors.py:12-17).
 */
#ifndef KM_KERNELS_H
#define KM_KERNELS_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { KM_OK = 0, KM_ERR_ARG = -1, KM_ERR_LAUNCH = -2, KM_ERR_UNSUPPORTED = -3 };
enum { KM_BF16 = 0, KM_F16 = 1, KM_F32 = 2 };          /* 16-bit activation / output dtypes */
enum { KM_Q_INT8 = 0, KM_Q_E4M3 = 1 };                  /* weight-only code formats */
enum { KM_WSCALE_ROWS = 0, KM_WSCALE_E8M0 = 1, KM_WSCALE_BLOCKS = 2 }; /* weight scale layouts of km_wo_gemm_dgrad_w16 */
enum { KM_SCALES_ROWMAJOR = 0, KM_SCALES_PACKED = 1, KM_SCALES_KMAJOR = 2 };  /* scale layouts the GEMMs read */
enum { KM_KERNEL_GEMM_MX = 0, KM_KERNEL_GEMM_FP8 = 1, KM_KERNEL_WO_FWD = 2, KM_KERNEL_WO_DGRAD = 3, KM_KERNEL_GEMM_BLOCKS = 4 };
enum { KM_ROLE_ACT = 0, KM_ROLE_WEIGHT = 1 };                     /* operand roles of the block recipe */

int km_abi_version(void);
const char *km_last_error(void);

/* MXFP8 quantizer of a logical [rows, cols] operand whose element (r, c) is at
 * x[r*stride_row + c*stride_col] (strides in elements; dtype KM_BF16 / KM_F16). Blocks of 32
 * run along cols (cols % 32 == 0). Writes q [rows, cols] e4m3fn bytes and the biased E8M0 scale
 * bytes in up to two layouts (either pointer may be NULL, not both): `scales` [rows, cols/32]
 * dense row-major (the reference's layout) and `scales_packed`, the MFMA-packed copy
 * km_gemm_mx reads fastest (cols % 128 == 0; km_scales_packed_bytes() bytes, the caller zero-
 * fills it first when rows % 128 != 0). A transposed view (stride_row == 1) is the reference's
 * column-wise quantization quantize(x.t(), "mx").
 * Replaces fp8.formats.quantize(x, "mx", role) (src/kohakumoss_kernels/fp8/formats.py:94-99),
 * Triton quantize_blocks(x, mx=True) (backends/triton/fp8/quantize.py:171-187) and, for the
 * packed output, Triton quantize_mx_swizzled (backends/triton/fp8/quantize.py:190-198). */
int km_quant_mx(const void *x, int64_t rows, int64_t cols, int64_t stride_row, int64_t stride_col,
                int dtype, void *q, void *scales, void *scales_packed, void *stream);

/* MFMA-packed copy of an MX scale matrix. For every K step of 128 columns and group of 128
 * rows it holds 512 bytes ordered [row % 16][block % 4][(row % 128) / 16]: byte (r, b) of the
 * natural [rows, cols/32] matrix sits at
 *   ((((b/4) * ceil(rows/128) + r/128) * 16 + r%16) * 4 + b%4) * 8 + (r%128)/16.
 * A lane of the block-scaled MFMA then finds the scales of the eight 16-row tiles of its
 * wavefront in 8 consecutive bytes and a wavefront reads them with one 512-byte load. It plays
 * the role of the vendor swizzle the reference keeps in `aux`
 * (swizzle_mx, src/kohakumoss_kernels/fp8/formats.py:128-136). Rows past `rows` are padding. */
int64_t km_scales_packed_bytes(int64_t rows, int64_t cols);
int km_scales_pack(const void *scales, int64_t rows, int64_t cols, void *out, void *stream);

/* Per-tensor e4m3 quantizer: *scale_out = max(amax, 1e-12) / 448 (IEEE division),
 * q = e4m3(clamp(x / scale)). amax_workspace is KM_QUANT_TENSOR_WORKSPACE_BYTES of device memory
 * (4-byte aligned, contents irrelevant) the call owns while it runs: the abs-max pass leaves one partial
 * maximum per work-group there and the conversion pass reduces them, so nothing has to be cleared and
 * no atomics are needed. Replaces fp8.formats.quantize(x, "tensor")
 * (src/kohakumoss_kernels/fp8/formats.py:77-79) and Triton quantize_tensor
 * (backends/triton/fp8/quantize.py:161-168). */
#define KM_QUANT_TENSOR_WORKSPACE_BYTES 2048
int km_quant_tensor(const void *x, int64_t rows, int64_t cols, int64_t stride_row, int64_t stride_col,
                    int dtype, void *q, float *scale_out, uint32_t *amax_workspace, void *stream);

/* Per-row e4m3 quantizer: scale_out[r] = max(amax of row r, 1e-12) / 448 (IEEE division),
 * q[r, :] = e4m3(clamp(x[r, :] / scale_out[r])) (IEEE division, clamp to +-448, one rounding).
 * Any strides and cols; unit-stride rows with cols % 8 == 0 take the vectorized kernel.
 * Replaces fp8.formats.quantize(x, "row") (src/kohakumoss_kernels/fp8/formats.py:80-82) and
 * Triton quantize_rows (backends/triton/fp8/quantize.py:64-84,151-158). */
int km_quant_rows(const void *x, int64_t rows, int64_t cols, int64_t stride_row, int64_t stride_col,
                  int dtype, void *q, float *scale_out, void *stream);

/* Block-recipe e4m3 quantizer (cols % 128 == 0, any strides). KM_ROLE_ACT: one scale per row and
 * 128 columns, scale_out [rows, cols/128] (the reference's layout) and / or scale_kmajor
 * [cols/128, rows], the copy km_gemm_fp8_blocks reads fastest (either may be NULL, not both);
 * KM_ROLE_WEIGHT: one scale per 128 x 128 block (rows past the end count as zeros), scale_out
 * [ceil(rows/128), cols/128], scale_kmajor NULL. scale = max(amax, 1e-12) / 448 and
 * q = e4m3(clamp(x / scale)), both IEEE divisions. q is [rows, cols] contiguous.
 * Replaces fp8.formats.quantize(x, "block", role) (src/kohakumoss_kernels/fp8/formats.py:83-93)
 * and, for activations, Triton quantize_blocks(x, mx=False) (backends/triton/fp8/quantize.py:95-119,
 * 171-187); the reference quantizes weight blocks with the eager formats only. */
int km_quant_blocks(const void *x, int64_t rows, int64_t cols, int64_t stride_row, int64_t stride_col,
                    int dtype, int role, void *q, float *scale_out, float *scale_kmajor, void *stream);

/* Per-row int8 quantizer of the int8 compute linear: v = x (* col_scale[c], in fp32, when col_scale
 * is not NULL; [cols] fp32), scale_out[r] = max(amax of row r of v, 1e-12) / 127 (IEEE division),
 * q[r, c] = clamp(round_half_even(v / scale_out[r]), +-127) (IEEE division). NaN inputs are outside
 * the contract. Replaces int8.formats.quantize_rows(x, col_scale)
 * (src/kohakumoss_kernels/int8/formats.py:21-38) and the Triton row quantizer
 * (backends/triton/int8.py). */
int km_quant_rows_i8(const void *x, int64_t rows, int64_t cols, int64_t stride_row, int64_t stride_col,
                     int dtype, const float *col_scale, void *q, float *scale_out, void *stream);

/* The same quantizer over the rotated activation, in one pass over x:
 * q, scale_out = quantize_rows(group_hadamard(x, group)), the rotation's result rounded to the
 * 16-bit type before it is quantized, exactly as km_group_hadamard followed by km_quant_rows_i8
 * gives it. Unit column stride, group >= 16, cols % group == 0, cols <= 4096, x and q 16-byte
 * aligned, stride_row % 8 == 0 (KM_ERR_UNSUPPORTED otherwise: run the two entry points instead). Replaces
 * the rotating form (G > 0) of the Triton row quantizer _quant_rows
 * (src/kohakumoss_kernels/backends/triton/int8.py:47-75). */
int km_quant_rows_i8_rotated(const void *x, int64_t rows, int64_t cols, int64_t stride_row, int dtype,
                             int group, void *q, float *scale_out, void *stream);

/* C[M,N] = (A .* 2^(a_scale-127)) (B .* 2^(b_scale-127))^T + bias, A [M,K] and B [N,K] e4m3fn
 * row-major (K contiguous), scales E8M0 bytes, both in the layout scale_layout names
 * (KM_SCALES_ROWMAJOR: [M,K/32] / [N,K/32]; KM_SCALES_PACKED: see km_scales_pack), fp32 accumulation
 * over all of K on the block-scaled MFMA, bias [N] (out_dtype, may be NULL) added in fp32, one
 * rounding to out_dtype. K % 128 == 0. config selects a tile configuration
 * (0 <= config < km_num_configs(KM_KERNEL_GEMM_MX)).
 * Replaces Triton dot_scaled_mm / promote_mm (backends/triton/fp8/gemm.py:108-171,219-231). */
int km_gemm_mx(const void *a, const void *a_scale, const void *b, const void *b_scale,
               const void *bias, void *c, int64_t M, int64_t N, int64_t K, int out_dtype,
               int scale_layout, int config, void *stream);

/* One-launch MXFP8 linear for short M: C[M,N] = Q(x) (B .* 2^(b_scale-127))^T + bias with x [M,K]
 * bf16 / fp16 (row pitch stride_row elements, unit column stride, 16-byte aligned rows) quantized
 * to MXFP8 inside the K loop with the arithmetic of km_quant_mx, B [N,K] e4m3fn, b_scale_packed its
 * MFMA-packed E8M0 scales (km_scales_pack), bias [N] and C in x's dtype. K % 128 == 0, N % 32 == 0.
 * Every workgroup quantizes its own rows of x again (N/64 times in all; N/32 when N % 64 != 0), so it
 * pays only where launches, not the MFMA, bound the linear: M up to about 32.
 * Replaces Triton fused_mx_mm (backends/triton/fp8/fused.py:98-120,182-194). */
int km_gemm_mx_fused(const void *x, int64_t stride_row, const void *b, const void *b_scale_packed,
                     const void *bias, void *c, int64_t M, int64_t N, int64_t K, int dtype, void *stream);

/* One-launch per-row fp8 linear for short M: C[m,n] = (Q(x) B^T)[m,n] * (s[m] * b_scale[n]) + bias[n],
 * s[m] = max(amax of row m of x, 1e-12) / 448 and Q(x) = e4m3(clamp(x / s[m])) taken inside the
 * kernel with the arithmetic of km_quant_rows (a prologue scans the rows for their abs-max), B [N,K]
 * e4m3fn, b_scale [N] fp32 (16-byte aligned). Same shape constraints and use as km_gemm_mx_fused.
 * Replaces Triton fused_row_mm (backends/triton/fp8/fused.py:35-68,152-165). */
int km_gemm_fp8_rows_fused(const void *x, int64_t stride_row, const void *b, const float *b_scale,
                           const void *bias, void *c, int64_t M, int64_t N, int64_t K, int dtype, void *stream);

/* One-launch block-recipe fp8 linear for short M: C[m,n] = sum over K blocks kb of (Q(x)[m,kb] . B[n,kb])
 * * s[m,kb] * b_scale[n/128,kb] + bias[n], with s[m,kb] = max(amax of x[m, 128 kb .. 128 kb + 127], 1e-12) / 448
 * and Q(x) = e4m3(clamp(x / s)) taken inside the kernel with the arithmetic of km_quant_blocks
 * (KM_ROLE_ACT); B [N,K] e4m3fn, b_scale [ceil(N/128), K/128] fp32. Same shape constraints and use as
 * km_gemm_mx_fused. Replaces Triton fused_block_mm (backends/triton/fp8/fused.py:71-95,167-179). */
int km_gemm_fp8_blocks_fused(const void *x, int64_t stride_row, const void *b, const float *b_scale,
                             const void *bias, void *c, int64_t M, int64_t N, int64_t K, int dtype, void *stream);

/* Per-tensor fp8 GEMM: C = (A B^T) * (*sa * *sb) + bias, sa / sb device fp32 scalars.
 * Replaces Triton scaled_mm for the tensor recipe (backends/triton/fp8/gemm.py:66-105,187-202)
 * and torch._scaled_mm (backends/triton/fp8/linear.py:121-130). K % 128 == 0. */
int km_gemm_fp8_tensor(const void *a, const float *sa, const void *b, const float *sb,
                       const void *bias, void *c, int64_t M, int64_t N, int64_t K, int out_dtype,
                       int config, void *stream);

/* Per-row fp8 GEMM: C[m,n] = (A B^T)[m,n] * (sa[m] * sb[n]) + bias[n], sa [M] and sb [N] device
 * fp32 vectors (sb 16-byte aligned). Replaces Triton scaled_mm for the row recipe
 * (backends/triton/fp8/gemm.py:66-105,187-202) and torch._scaled_mm with row-wise scales
 * (backends/triton/fp8/linear.py:130-136). K % 128 == 0. */
int km_gemm_fp8_rows(const void *a, const float *sa, const void *b, const float *sb,
                     const void *bias, void *c, int64_t M, int64_t N, int64_t K, int out_dtype,
                     int config, void *stream);

/* Block-recipe fp8 GEMM: C[m,n] = sum over K blocks kb of (A[m,kb] . B[n,kb]) * sa[m,kb] * sb[n/128,kb]
 * + bias[n]; sb [ceil(N/128), K/128] fp32; sa fp32 in the layout sa_layout names: KM_SCALES_ROWMAJOR
 * [M, K/128] or KM_SCALES_KMAJOR [K/128, M] (faster: the 16 rows of an MFMA tile read one run).
 * Each block's partial product is accumulated in fp32 on the MFMA and promoted (scaled and added
 * to the running fp32 sum) on the vector ALU. K % 128 == 0; config < km_num_configs(KM_KERNEL_GEMM_BLOCKS).
 * Replaces Triton promote_mm with sub = 128, b_rows = 128 (backends/triton/fp8/gemm.py:108-134,205-216). */
int km_gemm_fp8_blocks(const void *a, const float *sa, const void *b, const float *sb,
                       const void *bias, void *c, int64_t M, int64_t N, int64_t K, int out_dtype,
                       int sa_layout, int config, void *stream);

/* int8 GEMM with int32 accumulation: C[m,n] = ((float(A B^T)[m,n] * sa[m]) * sb[n]) + bias[n], every
 * product and the sum rounded to fp32 on its own and the result once to out_dtype, which makes
 * the output equal, bit for bit, to the reference's eager int8 linear. A [M,K] and B [N,K] int8
 * row-major, sa [M] fp32, sb [N] fp32 or NULL (ones; 16-byte aligned), bias [N] out_dtype or NULL.
 * K % 128 == 0. Forward: A = Q(x), B = q, sb = weight scales; int8 input gradient: A = Q(dy * scale),
 * B = q^T ([K,N] row-major copy), sb = NULL.
 * Replaces torch._int_mm + the fp32 epilogue of int8.op.fwd_reference / dgrad_reference
 * (src/kohakumoss_kernels/int8/op.py:40-60, int8/formats.py:39-52) and the Triton int8 GEMM
 * (backends/triton/int8.py:47-133). */
int km_gemm_i8_rows(const void *a, const float *sa, const void *b, const float *sb,
                    const void *bias, void *c, int64_t M, int64_t N, int64_t K, int out_dtype,
                    int config, void *stream);

/* Weight-only forward: y[M,N] = (x[M,K] @ q[N,K]^T) * scale[N] + bias[N]; q int8 or e4m3fn
 * widened exactly to the activation dtype in registers, fp32 accumulation, scale and bias on
 * the accumulator, one rounding. Replaces Triton _fwd_kernel (backends/triton/quant.py:27-77). */
int km_wo_gemm_fwd(const void *x, const void *q, const float *scale, const void *bias, void *y,
                   int64_t M, int64_t N, int64_t K, int q_format, int dtype, int config,
                   void *stream);

/* Weight-only input gradient: dx[M,K] = dy[M,N] @ round_dtype(q[N,K] * scale[N]); the scaled
 * weight tile is rounded once to the activation dtype, as dequantize-then-matmul does.
 * q_t_workspace is N*K bytes of device memory the call owns while it runs (the codes are
 * transposed into it so that the contraction axis N becomes contiguous).
 * Replaces Triton _dgrad_kernel (backends/triton/quant.py:80-129). */
int km_wo_gemm_dgrad(const void *dy, const void *q, const float *scale, void *dx,
                     void *q_t_workspace, int64_t M, int64_t N, int64_t K, int q_format, int dtype,
                     int config, void *stream);

/* Input gradient over the codes as they are stored, for int8 / e4m3 weight-only bases and for
 * fp8 compute bases that keep no transposed copy: dx[M,K] = dy[M,N] @ round_dtype(q[N,K] * s(n,k)),
 * the scaled weight rounded once to the activation dtype. The kernel transposes 8 x 4 bytes of
 * codes in registers on their way to LDS: no workspace, no transposed copy, nothing allocated.
 *   KM_WSCALE_ROWS    scale fp32 [N] (scale_ld 1) or one fp32 for the whole tensor (scale_ld 0)
 *   KM_WSCALE_E8M0    scale uint8 [N, scale_ld] biased exponents, one per 32 codes of a row (MX);
 *                     e4m3 codes only
 *   KM_WSCALE_BLOCKS  scale fp32 [ceil(N/128), scale_ld], one per 128 x 128 block; e4m3 codes only
 * Replaces Triton _dgrad_kernel (backends/triton/quant.py:80-129) and the 16-bit input gradient
 * `dy @ dequantize(q, scale)` of an fp8 base (backends/triton/fp8/linear.py:152-153 over
 * fp8/formats.py:103-126). */
int km_wo_gemm_dgrad_w16(const void *dy, const void *q, const void *scale, int scale_kind,
                         int64_t scale_ld, void *dx, int64_t M, int64_t N, int64_t K, int q_format,
                         int dtype, int config, void *stream);

/* km_wo_gemm_dgrad without a workspace argument and without any allocation: the transposed codes
 * go to a static device array of KM_WO_DGRAD_STATIC_MAX_CODES bytes that the library holds on every
 * GPU it runs on until the process ends. N*K beyond that is rejected (KM_ERR_UNSUPPORTED). Same
 * result as km_wo_gemm_dgrad, bit for bit. All calls on one GPU share the array: calls that overlap
 * on one GPU (two streams, two threads) race; calls on one stream are ordered and safe.
 * No counterpart in the reference: it is for callers that cannot allocate device memory around
 * the call (code under HIP graph capture, tight serving loops, harnesses that forbid it). */
#define KM_WO_DGRAD_STATIC_MAX_CODES (64ll << 20)
int km_wo_gemm_dgrad_static(const void *dy, const void *q, const float *scale, void *dx,
                            int64_t M, int64_t N, int64_t K, int q_format, int dtype, int config,
                            void *stream);

/* Which kernel class the weight-only entry points above would run for these operands: the tiled MFMA
 * kernels (KM_PATH_TILED) or the kernel with one thread per output element that serves every other
 * shape and alignment, correct and far slower (KM_PATH_ELEMENTWISE: K % 8 != 0 in forward; N % 8 != 0,
 * K % 4 != 0, operands not 16-byte aligned or extreme extents in the input gradient). Pointers are
 * only inspected for alignment. direction: KM_WO_FWD (a = x, c = y), KM_WO_DGRAD_W16 (a = dy, c = dx),
 * KM_WO_DGRAD_TRANSPOSED (km_wo_gemm_dgrad and km_wo_gemm_dgrad_static). A host layer uses it to tell
 * its caller about the slow path instead of timing it silently; no counterpart in the reference,
 * whose Triton kernels mask ragged tiles. */
enum { KM_WO_FWD = 0, KM_WO_DGRAD_W16 = 1, KM_WO_DGRAD_TRANSPOSED = 2 };
enum { KM_PATH_TILED = 0, KM_PATH_ELEMENTWISE = 1 };
int km_wo_gemm_path(int direction, const void *a, const void *q, const void *scale, const void *c,
                    int64_t M, int64_t N, int64_t K);

/* Group Hadamard rotation (ConvRot): y[r, :] = x[r, :] . blockdiag(H_group), H_group the normalised
 * Kronecker power of H4 = [[1,1,1,-1],[1,1,-1,1],[1,-1,1,1],[-1,1,1,1]] (symmetric, its own
 * inverse), group in {4, 16, 64, 256, 1024} dividing cols; x and y [rows, cols] contiguous,
 * 16-byte aligned, dtype KM_BF16 / KM_F16. fp32 4-point butterflies in the reference's stage
 * order, one scaling by 1/sqrt(group), one rounding. Replaces the Triton rotation
 * (backends/triton/hadamard.py:28-105) and hadamard.group_hadamard_eager
 * (src/kohakumoss_kernels/hadamard.py:71-101). */
int km_group_hadamard(const void *x, int64_t rows, int64_t cols, int dtype, int group, void *y,
                      void *stream);

/* Measurement only, no counterpart in the reference: the block-scaled fp8 MFMA run out of registers
 * (one wavefront per SIMD on every compute unit, 64 independent 16x16x128 MFMAs per trip over eight
 * fragments of each operand, no loads, no LDS, no barriers), `trips` trips per wavefront. a_frags and
 * b_frags are 16 KiB of e4m3 codes each (8 fragments x 64 lanes x 32 bytes, 32-byte aligned): a
 * benchmark passes rows of its real operands so that the data-dependent power draw matches. sink
 * takes 256 floats per compute unit. *flop_out receives the launch's flop count; flop / device
 * time is the rate the card's clocks sustain on its matrix pipes, the ceiling of the GEMMs above
 * (the method of the reference's docs/performance/gemm-efficiency.md:28-29: peak from the measured
 * clock, not the nominal one). */
int km_probe_mfma_ceiling(const void *a_frags, const void *b_frags, void *sink, int64_t sink_floats,
                          int trips, int64_t *flop_out, void *stream);

/* Tile configurations per kernel, for the host-side tuning table (the reference enumerates its
 * Triton tiles in backends/triton/fp8/linear.py:39-75 and backends/triton/quant.py:132-141).
 * km_config_desc writes "key=value,..." (bm, bn: rows and columns of a work-group's tile; for the
 * weight-only kernels tail=1 means that a second launch puts half-size tiles over the tile columns
 * which whole rounds of the card's compute units leave over). */
int km_num_configs(int kernel);
int km_config_desc(int kernel, int config, char *buf, int len);

#ifdef __cplusplus
}
#endif
#endif
