/*
 * metis_hip.h -- C ABI of libmetis_hip.so: the Metis NVFP4 hot path as HIP kernels for gfx950.
 *
 * The reference implements this path as eager PyTorch code with no native entry points, so each
 * function below names the Python function whose arithmetic it replaces (paths relative to the
 * reference checkout).  A binding needs nothing but device pointers, sizes and a stream.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless stated otherwise; `stream` is a hipStream_t
 *     passed as void* (NULL = the default stream)
 *   - tensors are row-major; bf16 tensors are 16-bit patterns
 *   - functions enqueue work on `stream` and return immediately; they never allocate, free or
 *     synchronise.  Scratch memory comes from the caller (`workspace`), must be 256-byte
 *     aligned, zero-filled once when it is allocated, and may be reused by later calls on the
 *     same stream (calls that share a workspace must not overlap in time)
 *   - return value: METIS_OK or a negative METIS_E_* code; nothing is written on error
 *   - `mode` selects which arithmetic of the reference is reproduced bit for bit:
 *       METIS_MODE_P32  binary32 arithmetic on the bf16-valued input (reference run with
 *                       compute_dtype=float32, src/Metis/Metis/bitlinear.py:70,377)
 *       METIS_MODE_PB16 every eager op rounded to bf16 (compute_dtype=bfloat16,
 *                       src/grpo/grpo.py:204-205)
 *       METIS_MODE_P32_F32  (metis_nvfp4_quant_* only) binary32 arithmetic on a binary32 tensor whose
 *                       values need not be bf16 values: gradients and activations downstream of a
 *                       layer that ran with compute_dtype=float32 (src/dpo/run_dpo_metis.py:134;
 *                       the forward returns binary32, src/Metis/Metis/bitlinear.py:435-441).  x is
 *                       float [rows, cols] (row stride ld % 4 == 0), noise float; the packed result
 *                       is an ordinary METIS_MODE_P32 tensor.
 *
 * NVFP4 layout produced / consumed (the reference never materialises it; these are the integers
 * its arithmetic passes through, src/Metis/Metis/quant.py:19-31)
 *   codes  uint8 [rows, cols/2]   element 2j in the low nibble of byte j;
 *                                 nibble = (x < 0) << 3 | r, r in 0..7 the E2M1 magnitude code
 *   scales uint8 [rows, cols/16]  float8_e4m3fn byte of (block scalar / unit)
 *   unit   float                  max(block scalar) / 448   (bf16-valued in METIS_MODE_PB16)
 *   value of an element = e2m1(r) * sign * e4m3(scale) * unit,  e2m1 = {0,.5,1,1.5,2,3,4,6}
 */
#ifndef METIS_HIP_H
#define METIS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define METIS_OK 0
#define METIS_E_ARG (-1)       /* null pointer, negative size, unknown mode/dtype             */
#define METIS_E_SHAPE (-2)     /* block of 16 does not divide the blocked dimension -> ValueError
                                  in the reference (src/Metis/Metis/quant.py:400-403)          */
#define METIS_E_WORKSPACE (-3) /* workspace missing, misaligned or too small                   */
#define METIS_E_LAUNCH (-4)    /* the HIP runtime rejected a launch                             */
#define METIS_E_DEVICE (-5)    /* not a gfx950 device / required feature missing               */
#define METIS_E_TOO_LARGE (-6) /* metis_nvfp4_quant_row_static: more elements than its scratch holds */

#define METIS_MODE_P32 0
#define METIS_MODE_PB16 1
#define METIS_MODE_P32_F32 2   /* quantizer entry points only: METIS_MODE_P32 with x (and noise) binary32 */

#define METIS_DTYPE_BF16 0
#define METIS_DTYPE_F32 1

/* Library version, (major << 16) | (minor << 8) | patch.  No reference counterpart. */
int metis_version(void);

/* Static text for a return code.  Host pointer, never NULL. */
const char *metis_error_string(int code);

/* Bytes of workspace the quantizer entry points need for a [rows, cols] tensor. */
size_t metis_nvfp4_workspace_bytes(int64_t rows, int64_t cols);

/*
 * NVFP4 round-to-nearest quantizer, blocks of 16 along the last dimension.
 * Replaces Cast2NVFp4e2m1BlockNOSR.quantize_dequantize -> _nvfp4_nosr_quantize_dequantize
 * (src/Metis/Metis/quant.py:6-36, 392-433) up to the dequantisation, i.e. it emits the packed
 * integers; metis_nvfp4_dequant() completes the round trip.
 *   x      bf16 [rows, cols], row stride `ld` elements (ld >= cols)
 *   codes  uint8 [rows, cols/2]; scales uint8 [rows, cols/16]; unit float[1]
 * METIS_E_SHAPE when cols % 16 != 0.
 */
int metis_nvfp4_quant_row(const void *x, int64_t rows, int64_t cols, int64_t ld, int mode,
                          void *codes, void *scales, float *unit, void *workspace,
                          size_t workspace_bytes, void *stream);

/*
 * The quantize -> dequantize round trip of _nvfp4_nosr_quantize_dequantize (src/Metis/Metis/quant.py:6-36) with all
 * three of its results from one call: packed codes, E4M3 scale bytes + unit, and the dequantized tensor
 * out = ((v * sign) / 2) * (e4m3 * unit) (quant.py:23-26, 32-35) in bf16.  Two launches: phase 1 of
 * metis_nvfp4_quant_row, then one pass over the codes and the parked block maxima that forms scale bytes and
 * dequantized values together.  Same bytes as metis_nvfp4_quant_row followed by metis_nvfp4_dequant.
 *   x      bf16 [rows, cols], contiguous
 *   out    bf16 [rows, cols]
 *   mode   METIS_MODE_P32 or METIS_MODE_PB16
 */
int metis_nvfp4_quant_dequant_row(const void *x, int64_t rows, int64_t cols, int mode, void *codes,
                                  void *scales, float *unit, void *out, void *workspace,
                                  size_t workspace_bytes, void *stream);

/*
 * metis_nvfp4_quant_row without a workspace argument and without any allocation: the scratch (per-workgroup
 * maxima and the parked block maxima) is a static device array inside the library.  No counterpart in the
 * reference; it exists for callers that cannot allocate device memory: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  Same kernels and same bytes as metis_nvfp4_quant_row.
 *   limit   rows * cols <= 2^26 elements (METIS_E_TOO_LARGE beyond that; nothing is launched)
 *   cost    every device the library runs on holds the 16.1 MiB array from first use until the process ends
 *   sharing all calls on one device use that device's single array: calls that overlap in time on one
 *           device (two streams, two host threads) race on it and must be ordered by the caller
 * The call never calls hipMalloc/hipFree or any allocating routine; its first call on a device looks the
 * array's address up once (hipGetSymbolAddress, which may load the code object and place the array) and reads a few
 * device properties: make that FIRST call per device outside stream capture (any size, e.g. at start-up).  Every later
 * call only launches two kernels and may be captured into a HIP graph (no memset node is recorded).
 */
int metis_nvfp4_quant_row_static(const void *x, int64_t rows, int64_t cols, int64_t ld, int mode,
                                 void *codes, void *scales, float *unit, void *stream);

/*
 * metis_nvfp4_quant_row (contiguous rows, round to nearest) as ONE launch: block maxima stay in registers across a
 * grid-wide maximum taken through a small tree of device-scope atomics in the workspace, so in the ordinary case
 * neither the parked maxima nor the second kernel are needed.  Same bytes as metis_nvfp4_quant_row, always: a
 * workgroup that has polled for the grid's maximum `spin_limit` times (0 = the default of 4096, a few milliseconds)
 * without seeing it -- because part of the grid still waits for a compute unit that another kernel, or these very
 * pollers, hold -- parks its block maxima, leaves, and the last workgroup to arrive writes its scale bytes for it.
 * Every wave exits after a bounded time whatever else runs on the device.  Tensors too large for one launch of at
 * most 4096 workgroups with 8 blocks per thread take the two-launch path.
 * The workspace's reduction area (see metis_nvfp4_workspace_bytes) must be zero when first used and must not be
 * shared by calls that overlap in time; a call leaves it ready for the next one.  Measured on MI355X the single
 * launch is as fast as the two launches, not faster (the atomics' round trips cost what the second launch costs), so
 * it is not the default.  Same arithmetic as quant.py:6-36; the reference has no counterpart for the launch structure.
 */
int metis_nvfp4_quant_row_resident(const void *x, int64_t rows, int64_t cols, int mode, void *codes,
                                   void *scales, float *unit, void *workspace, size_t workspace_bytes,
                                   uint32_t spin_limit, void *stream);

/*
 * Same quantizer with blocks of 16 along dimension 0 (tokens), written transposed: the operand
 * layout of a GEMM that contracts over tokens.  Equals metis_nvfp4_quant_row applied to x^T.
 * The reference quantizes dY along its last dimension only (src/Metis/Metis/bitlinear.py:
 * 395-405, 488-492), which a block-scaled GEMM cannot contract over tokens.
 *   x      bf16 [rows, cols], row stride ld
 *   codes  uint8 [cols, rows/2]; scales uint8 [cols, rows/16]; unit float[1]
 * METIS_E_SHAPE when rows % 16 != 0.
 */
int metis_nvfp4_quant_col(const void *x, int64_t rows, int64_t cols, int64_t ld, int mode,
                          void *codes, void *scales, float *unit, void *workspace,
                          size_t workspace_bytes, void *stream);

/*
 * NVFP4 stochastic-rounding quantizer: Cast2NVFp4e2m1Block.get_scalar/quant
 * (src/Metis/Metis/quant.py:273-308) with the element rule of Cast2Fp4e2m1Random.quant
 * (137-147): compress, add (u - 0.5), round.
 *   noise  the uniform draws in [0,1) to use, same shape as x: float32 in METIS_MODE_P32, bf16 in
 *          METIS_MODE_PB16 (what torch.rand_like yields for that dtype): the reference's op sequence
 *          is followed literally and the result is bit-exact for shared draws.  A draw that rounds
 *          the block maximum up to r = 8 (possible in the reference, which then returns the
 *          off-grid value 8 * scalar) is clamped to r = 7.
 *          NULL -> the library's own stream: one Philox4x32-10 draw per output block (counter =
 *          offset + block index in the packed orientation, key = seed) feeds the hardware
 *          stochastic-rounding converter.  Same distribution (P(up) = position between the two
 *          neighbouring grid points), about 2.5x faster, not comparable draw by draw with torch's
 *          generator; a call consumes rows * cols / 16 counters.
 * Scale bytes and unit do not depend on the rounding mode.
 */
int metis_nvfp4_quant_sr_row(const void *x, int64_t rows, int64_t cols, int64_t ld, int mode,
                             const void *noise, uint64_t seed, uint64_t offset, void *codes,
                             void *scales, float *unit, void *workspace, size_t workspace_bytes,
                             void *stream);

/* Column-blocked stochastic rounding: metis_nvfp4_quant_sr_row of x^T; `noise`, when given, is
 * indexed like x (noise[r, c] belongs to x[r, c]); the library's own stream is indexed by the blocks of x^T. */
int metis_nvfp4_quant_sr_col(const void *x, int64_t rows, int64_t cols, int64_t ld, int mode,
                             const void *noise, uint64_t seed, uint64_t offset, void *codes,
                             void *scales, float *unit, void *workspace, size_t workspace_bytes,
                             void *stream);

/*
 * Both packings of one tensor with stochastic rounding on the library's own stream, in one pass over x: the
 * backward pass needs dY blocked along its last dimension for dX = dY W and blocked down its columns for
 * dW = dY^T X (src/Metis/Metis/bitlinear.py:488-510 quantizes grad_output for each product).  The results are
 * those of metis_nvfp4_quant_sr_row(.., noise = NULL, seed, offset_row, ..) and metis_nvfp4_quant_sr_col(.., noise =
 * NULL, seed, offset_col, ..), byte for byte; each consumes rows * cols / 16 counters from its own offset.
 *   x          bf16 [rows, cols] (binary32 in METIS_MODE_P32_F32), row stride ld (ld % 8 == 0, ld % 4 in binary32),
 *              16-byte aligned; rows % 16 == 0 and cols % 16 == 0, else METIS_E_SHAPE
 *   workspace  2 * metis_nvfp4_workspace_bytes(rows, cols) bytes
 */
int metis_nvfp4_quant_sr_both(const void *x, int64_t rows, int64_t cols, int64_t ld, int mode,
                              uint64_t seed, uint64_t offset_row, uint64_t offset_col,
                              void *codes_row, void *scales_row, float *unit_row, void *codes_col,
                              void *scales_col, float *unit_col, void *workspace,
                              size_t workspace_bytes, void *stream);

/*
 * The reference's three-call form on dequantized tensors of dtype D (float32 in METIS_MODE_P32, bf16 in
 * METIS_MODE_PB16), for callers that use the quantizer classes directly.  All tensors contiguous [rows, cols].
 *   metis_nvfp4_get_scalar : Cast2NVFp4e2m1Block[NOSR].get_scalar (src/Metis/Metis/quant.py:435-455)
 *                            s [rows, cols/16] = amax|x| / 6 + 1e-9
 *   metis_nvfp4_quant_values : .quant (quant.py:459-466; element rule 118-128, or 137-147 when sr != 0)
 *                            out [rows, cols] in {0, +-0.5, ..., +-6} (+-8 possible under sr, as in the reference)
 *   metis_nvfp4_rquant     : .rquant (quant.py:470-548): s is DIVIDED IN PLACE by max|s|/448 as the reference
 *                            does; out = xq * (e4m3_roundtrip(s) * max|s|/448).  scratch: float[1] on the device.
 */
int metis_nvfp4_get_scalar(const void *x, int64_t rows, int64_t cols, int mode, void *s, void *stream);
int metis_nvfp4_quant_values(const void *x, const void *s, int64_t rows, int64_t cols, int mode, int sr,
                             const void *noise, uint64_t seed, uint64_t offset, void *out, void *stream);
int metis_nvfp4_rquant(const void *xq, void *s, int64_t rows, int64_t cols, int mode, void *out, float *scratch,
                       void *stream);

/*
 * Dequantize packed NVFP4: the last three multiplications of the reference,
 * out = ((v * sign) / 2) * (e4m3 * unit)  (src/Metis/Metis/quant.py:23-24, 32-35; rquant 470-548).
 *   out    [rows, cols] of out_dtype (METIS_DTYPE_BF16 or METIS_DTYPE_F32); in METIS_MODE_P32 a
 *          bf16 output is the binary32 result rounded once
 */
int metis_nvfp4_dequant(const void *codes, const void *scales, const float *unit, int64_t rows,
                        int64_t cols, int mode, void *out, int out_dtype, void *stream);

/*
 * Fused RMSNorm -> NVFP4 quantization of the normed activations: one read of the hidden states.
 * RMSNorm follows src/Metis/models/llama.py:23-31 with a bf16 weight (binary32 normalisation,
 * rounded to bf16, times gamma, rounded to bf16); the quantizer is metis_nvfp4_quant_row applied
 * to the bf16 normed values.  The reference has no fused op: it runs the norm, then quantizes
 * in LinearLowbitFunction.quantize_input (src/Metis/Metis/bitlinear.py:371-393).
 *   x      bf16 [rows, cols]; gamma bf16 [cols]
 *   normed bf16 [rows, cols] (may be NULL when only the packed form is wanted)
 */
int metis_rmsnorm_nvfp4_quant(const void *x, const void *gamma, float eps, int64_t rows,
                              int64_t cols, int mode, void *normed, void *codes, void *scales,
                              float *unit, void *workspace, size_t workspace_bytes, void *stream);

/*
 * RMSNorm for the mean mode, the reference's default arguments (src/grpo/grpo.py:66-69): there the activation that
 * enters a projection group is quantized as mean + QDQ(x - mean) with the column mean over tokens
 * (src/Metis/Metis/bitlinear.py:311-336), so the quantizer cannot start before the whole normed tensor's mean is
 * known.  This call is the norm of metis_rmsnorm_nvfp4_quant (same arithmetic, src/Metis/models/llama.py:23-31) and
 * hands back the normed bf16 tensor together with its column mean -- `input_flat.mean(dim=0)` of bitlinear.py:326,
 * binary32 sums in a fixed order -- from one pass over x; metis_nvfp4_quant_centered then takes normed and mean.
 *   x       bf16 [rows, cols], cols <= 4096 and a multiple of 16; gamma bf16 [cols]
 *   normed  bf16 [rows, cols]
 *   mean    [cols] in mean_dtype (METIS_DTYPE_F32 for binary32 arithmetic, METIS_DTYPE_BF16 for bf16 arithmetic: the
 *           division by rows and every later operation are rounded to it)
 *   cached, cached_count   (optional) the weighted running mean of single-token decode calls, bitlinear.py:316-323:
 *           mean = (cached * cached_count + this_mean * rows) / (cached_count + rows)
 *   mean32  (optional) the same values once more as binary32
 *   workspace   metis_rmsnorm_colmean_workspace_bytes(rows, cols) bytes, 16-byte aligned, no initialisation needed
 */
size_t metis_rmsnorm_colmean_workspace_bytes(int64_t rows, int64_t cols);
int metis_rmsnorm_colmean(const void *x, const void *gamma, float eps, int64_t rows, int64_t cols,
                          void *normed, void *mean, int mean_dtype, const void *cached,
                          int64_t cached_count, float *mean32, void *workspace, size_t workspace_bytes,
                          void *stream);

/*
 * Block-scaled NVFP4 GEMM with an optional bf16 low-rank extension and bias:
 *   out[M,N] = ua*ub * sum_k deq(A)[m,k] * deq(B)[n,k]  +  sum_j T[m,j] * U[n,j]  +  bias[n]
 * A (M x K) and B (N x K) are packed NVFP4 with blocks of 16 along K; *ua, *ub are their units.
 * Products of E2M1 and E4M3 values are exact in bf16, accumulation is binary32 (MFMA).
 * Replaces torch.matmul(input_, quantized_weight.T) (+ bias) in LinearLowbitFunction.forward
 * (src/Metis/Metis/bitlinear.py:435-438) and, with T = (X V^T) * s and U, the sum of the two
 * branches in BitLinear.forward (src/Metis/Metis/bitlinear.py:752-760).
 *   t      bf16 [M, r] row stride r, u bf16 [N, r]; r % 32 == 0 or r == 0 (t, u NULL)
 *   bias   bf16 [N] or NULL
 *   out    [M, N] of out_dtype
 */
int metis_linear_fwd(const void *a_codes, const void *a_scales, const float *a_unit,
                     const void *b_codes, const void *b_scales, const float *b_unit, int64_t M,
                     int64_t N, int64_t K, const void *t, const void *u, int64_t r,
                     const void *bias, void *out, int out_dtype, void *stream);

/*
 * Expanded operands for compute-bound shapes.  metis_nvfp4_expand_f16 writes, for a packed tensor,
 *   out[i,k] = e2m1(code) * e4m3(scale) * 2^-8   as binary16 [rows, cols]   (exact; unit not applied)
 * and metis_linear_fwd_expanded computes the same result as metis_linear_fwd from two such tensors and
 * the two units (it multiplies the accumulators by unit_a * unit_b * 2^16).  The inner loop then is MFMA
 * and LDS reads only; the expansion costs 2 B/element of HBM and can be cached with a weight, as the
 * reference caches its dequantized weight (src/Metis/Metis/bitlinear.py:563-589).
 * Limits: K % 64 == 0, N % 4 == 0, r % 32 == 0.
 */
int metis_nvfp4_expand_f16(const void *codes, const void *scales, int64_t rows, int64_t cols, void *out,
                           void *stream);
int metis_linear_fwd_expanded(const void *a_exp, const float *a_unit, const void *b_exp, const float *b_unit,
                              int64_t M, int64_t N, int64_t K, const void *t, const void *u, int64_t r,
                              const void *bias, void *out, int out_dtype, void *stream);

/*
 * Expansion of a packed tensor into the layout the pipelined GEMM streams from, and that GEMM.
 * Layout: tiles of 16 rows x 32 k (1 KiB each, tile (rb, kb) at byte ((rb * cols/32) + kb) * 1024, rows padded to a
 * multiple of 16 with zeros), the 16-byte chunks of a tile permuted so that one direct-to-LDS load per tile leaves
 * it free of bank conflicts for the MFMA fragment reads.  Element values by `mode`:
 *   METIS_MODE_P32   binary16  e2m1(code) * e4m3(scale) * 2^-8, exact; the GEMM applies unit_a * unit_b * 2^16 to its
 *                    accumulators.  Results equal metis_linear_fwd on the packed operands bit for bit when neither
 *                    splits K (same exact products, same order of binary32 accumulation).
 *   METIS_MODE_PB16  bf16, the value the reference's quantize_dequantize returns when every op rounds to bf16
 *                    (src/Metis/Metis/quant.py:23-24, 32-35: bf16(bf16(e4m3 * unit) * v / 2), `unit` required), and the
 *                    GEMM follows the reference's all-bf16 forward (src/Metis/Metis/bitlinear.py:435-438 with
 *                    compute_dtype = bfloat16, as src/grpo/grpo.py:204-205 configures it): bf16 operands, binary32
 *                    accumulation, the residual product rounded to bf16, the bias added in bf16, then the low-rank
 *                    term t u^T (binary32) and one final rounding to bf16 (a binary32 `out` receives those bf16 values).
 *                    Both operands must have been packed and expanded in this mode; the units are not read.
 * metis_linear_fwd_tiled runs a main loop of MFMA and LDS reads only, its operand tiles arriving through a ring of
 * direct-to-LDS loads.  Derived data like the expansion above: callers cache a weight's tiled expansion next to its
 * packed form and re-expand an activation per call (2.56 B/element).  With a workspace
 * (metis_linear_tiled_workspace_bytes, 16-byte aligned, no initialisation; 0 = the shape is not split; NULL = never
 * split) shapes with few 256 x 256 output tiles split K as metis_linear_fwd_ws does.
 *   limits  cols % 32 == 0; GEMM: K % 32 == 0, N % 4 == 0, r % 32 == 0; out, t, u 16-byte aligned
 *   bias    bf16 [N], or float [N] when bias_is_f32 != 0, or NULL
 */
size_t metis_nvfp4_expand_tiled_bytes(int64_t rows, int64_t cols);
int metis_nvfp4_expand_tiled(const void *codes, const void *scales, const float *unit, int64_t rows,
                             int64_t cols, int mode, void *out, void *stream);
size_t metis_linear_tiled_workspace_bytes(int64_t M, int64_t N, int64_t K, int mode);

/*
 * A dense tensor as a tiled GEMM operand: x [rows, cols] bf16 or float (dtype METIS_DTYPE_*, row stride ld) in the layout
 * of metis_nvfp4_expand_tiled, each value rounded once to binary16 (mode METIS_MODE_P32; pass a device float 2^-8 as this
 * operand's unit to metis_linear_fwd_tiled, which multiplies by 2^16 for two exact expansions) or to bf16
 * (METIS_MODE_PB16).  col_scale (bf16 [cols], 16-byte aligned, or NULL) multiplies column k first, rounded to x's dtype.
 * For the merged rollout forward of src/Metis/Metis/bitlinear.py:705-751: the merged weight
 * (U diag(s)) Q(V) + Q(W_res) is a dense matrix, and the rollout multiplies the dequantized activation by it --
 * here metis_linear_fwd_tiled on the activation's tiled expansion and this operand.
 *   limits  cols % 32 == 0; x and out 16-byte aligned; ld % 8 == 0 (bf16) or % 4 (float); out holds
 *           metis_nvfp4_expand_tiled_bytes(rows, cols) bytes
 */
int metis_dense_expand_tiled(const void *x, int64_t rows, int64_t cols, int64_t ld, int dtype,
                             const void *col_scale, int mode, void *out, void *stream);

/*
 * NV recipe (tiled random Hadamard rotation, tile = 16 = the scale block) on the packed kernels.
 * The reference rotates a tensor tile by tile along its last dimension, (x * sign) H with the Sylvester matrix H_16 and
 * one shared sign vector (src/Metis/Metis/bitlinear.py:75-137, 199-202), quantizes and dequantizes the rotated tensor,
 * and rotates back, (q H) / 16 * sign (195-197): `_quantize_wgrad_operand` (395-405) for dY and X of the weight
 * gradient (495-501) and `_get_quantized_weight` (577-585) for the forward weight.  `sign_mask` carries the sign
 * vector: bit j set <=> sign[j] = -1 (the reference draws it with torch.randint under seed 1729 + 16; the Python host
 * side reproduces that draw and passes the mask).
 *   metis_hadamard16            the rotation (inverse != 0: the rotation back) of a bf16 or float tensor, same dtype out;
 *                               binary32 sums in butterfly order, one rounding to the output dtype
 *   metis_nvfp4_quant_row_rht   rotation and row quantizer in one pass over x: the packed tensor holds QDQ's codes of
 *                               the ROTATED tensor.  mode as metis_nvfp4_quant_row (bf16 arithmetic rounds the rotated
 *                               values to bf16 first, as the reference's bf16 tensor does); sr != 0: stochastic
 *                               rounding on the library's own stream (seed, offset) as metis_nvfp4_quant_sr_row
 *                               without caller noise
 *   metis_nvfp4_expand_tiled_rht  metis_nvfp4_expand_tiled of such a packed tensor with the rotation back applied to
 *                               every dequantized block (rotate_back != 0), so that the tiled operand holds the values
 *                               the reference multiplies with; mode METIS_MODE_P32: one rounding to binary16 (a block's
 *                               rotated sum needs at most 12 significant bits; relative error <= 2^-12), tensor unit
 *                               left to the GEMM; METIS_MODE_PB16: dequantized values and result rounded to bf16.
 *                               transpose != 0: the tiled operand of the TRANSPOSED tensor, [cols, rows] with the
 *                               contraction over rows (rows % 32 == 0): what the weight-gradient GEMM (contraction over
 *                               tokens) and the input-gradient GEMM (contraction over out_features) read;
 *                               out holds metis_nvfp4_expand_tiled_bytes(cols, rows) bytes then
 *   limits  cols % 16 == 0 (expand: cols % 32 == 0 when not transposed); 16-byte aligned x / out, ld % 8 == 0 (bf16)
 */
int metis_hadamard16(const void *x, int64_t rows, int64_t cols, int64_t ldx, int dtype, int inverse,
                     uint32_t sign_mask, void *out, int64_t ldo, void *stream);
int metis_nvfp4_quant_row_rht(const void *x, int64_t rows, int64_t cols, int64_t ld, int mode,
                              uint32_t sign_mask, int sr, uint64_t seed, uint64_t offset, void *codes,
                              void *scales, float *unit, void *workspace, size_t workspace_bytes,
                              void *stream);
int metis_nvfp4_expand_tiled_rht(const void *codes, const void *scales, const float *unit, int64_t rows,
                                 int64_t cols, int mode, uint32_t sign_mask, int rotate_back,
                                 int transpose, void *out, void *stream);
/*
 * Deferred scale bytes.  The codes of a block depend on the block alone (src/Metis/Metis/quant.py:27), the E4M3 bytes
 * and the tensor unit on the maximum over the whole tensor (quant.py:21-23) -- which is why the quantizers above are two
 * launches.  A consumer that runs after the quantizer anyway can form the bytes itself, so these entry points stop
 * after the first launch and park what the second would have read in a buffer the CALLER owns (it travels with the
 * codes): 2048 partial tensor maxima, then one bf16 block maximum per block.  Round-to-nearest rows of a contiguous
 * bf16 tensor (ld == cols), mode METIS_MODE_P32 or METIS_MODE_PB16.
 *   metis_nvfp4_deferred_bytes           size of that buffer; 256-byte aligned, contents need no initialisation
 *   metis_nvfp4_quant_row_deferred       metis_nvfp4_quant_row without scales and unit; center: NULL, or in mode
 *                                        METIS_MODE_PB16 one bf16 value per column subtracted first (16-byte aligned), as
 *                                        metis_nvfp4_quant_centered does for the mean mode
 *   metis_rmsnorm_nvfp4_quant_deferred   metis_rmsnorm_nvfp4_quant likewise
 *   metis_nvfp4_expand_tiled_deferred    metis_nvfp4_expand_tiled reading the parked data: quant_mode = the mode of the
 *                                        quantizer call, mode = the operand format; center: NULL, or (mode
 *                                        METIS_MODE_PB16) the bf16 centre as in metis_nvfp4_expand_tiled_centered; also
 *                                        writes the tensor unit (float [1], required), which metis_linear_fwd_tiled
 *                                        reads afterwards.  Same bits as
 *                                        the two-launch quantizer followed by metis_nvfp4_expand_tiled
 *   metis_nvfp4_deferred_scales          the second launch after all: scales and unit exactly as metis_nvfp4_quant_row
 *                                        would have written them, for consumers that read E4M3 bytes
 */
size_t metis_nvfp4_deferred_bytes(int64_t rows, int64_t cols);
int metis_nvfp4_quant_row_deferred(const void *x, int64_t rows, int64_t cols, int mode, const void *center,
                                   void *codes, void *deferred, size_t deferred_bytes, void *stream);
int metis_rmsnorm_nvfp4_quant_deferred(const void *x, const void *gamma, float eps, int64_t rows, int64_t cols,
                                       int mode, void *normed, void *codes, void *deferred,
                                       size_t deferred_bytes, void *stream);
int metis_nvfp4_expand_tiled_deferred(const void *codes, const void *deferred, int64_t rows, int64_t cols,
                                      int quant_mode, int mode, const void *center, float *unit, void *out,
                                      void *stream);
int metis_nvfp4_deferred_scales(const void *deferred, int64_t rows, int64_t cols, int mode, void *scales,
                                float *unit, void *stream);

/*
 * "svd" mode of the activation / output-gradient decomposition (LinearLowbitFunction.svd_quant with metis_mode = "svd",
 * src/Metis/Metis/bitlinear.py:243-309): with the factors of a rank-r approximation in hand (torch.svd_lowrank, U and V
 * through the three-call QDQ, :270-293), the reference forms ker = U diag(s) V (:296), quantizes x - ker (:300-301) and
 * goes on with ker + QDQ(x - ker) (:303).  This call does the three steps without storing ker or the residual: ker is
 * formed tile by tile in registers, the residual is encoded there, and the dense sum is written only when asked for.
 *   x        [rows, cols] contiguous: bf16, or (mode METIS_MODE_P32 only) binary32 with x_dtype = METIS_DTYPE_F32
 *   us       [rows, rank]  U diag(s), i.e. `ug @ torch.diag(sg)`: binary32 (METIS_MODE_P32) or bf16 (METIS_MODE_PB16)
 *   vt       [rank, cols]  V after `vg = vg.T`, same type as us
 *   mode     METIS_MODE_P32: everything in binary32 (compute_dtype = float32); METIS_MODE_PB16: ker rounded to bf16 once
 *            after binary32 accumulation, the subtraction and the quantizer in bf16 arithmetic
 *   codes, scales, unit   the packed residual QDQ(x - ker), as metis_nvfp4_quant_row writes them
 *   dense    NULL, or [rows, cols] in the arithmetic's type (binary32 / bf16): receives ker + QDQ(x - ker)
 *   workspace  metis_nvfp4_workspace_bytes(rows, cols)
 * Every element of ker is the chain acc = fma(us[i][k], vt[k][j], acc) over k = 0 .. rank-1 in that order in binary32
 * (a library matrix product sums in an order of its own: results agree to rounding, not to the bit).
 * Limits: cols % 16 == 0, rank % 16 == 0, 16-byte aligned tensors.  Two launches, three with dense.
 */
int metis_nvfp4_quant_lowrank_residual(const void *x, int x_dtype, const void *us, const void *vt,
                                       int64_t rows, int64_t cols, int rank, int mode, void *codes,
                                       void *scales, float *unit, void *dense, void *workspace,
                                       size_t workspace_bytes, void *stream);

/*
 * Mean mode in bf16 arithmetic: the activation the reference multiplies with is X^ = me + QDQ(X - me) as ONE bf16
 * tensor, the sum rounded to bf16 (LinearLowbitFunction.svd_quant with metis_mode = "mean",
 * src/Metis/Metis/bitlinear.py:311-336, under compute_dtype = bfloat16).  This is metis_nvfp4_expand_tiled with
 * mode = METIS_MODE_PB16 of the packed centred residual (metis_nvfp4_quant_centered) with that sum applied: the
 * tiled operand holds X^ itself, and metis_linear_fwd_tiled with mode = METIS_MODE_PB16 then follows the reference's
 * all-bf16 forward without a separate W^ me term.
 *   center  bf16 [cols], 16-byte aligned (required)
 */
int metis_nvfp4_expand_tiled_centered(const void *codes, const void *scales, const float *unit, int64_t rows,
                                      int64_t cols, const void *center, void *out, void *stream);
int metis_linear_fwd_tiled(const void *a_xt, const float *a_unit, const void *b_xt, const float *b_unit,
                           int64_t M, int64_t N, int64_t K, const void *t, const void *u, int64_t r,
                           const void *bias, int bias_is_f32, void *out, int out_dtype, int mode,
                           void *workspace, size_t workspace_bytes, void *stream);

/*
 * grad_input[L,K] = deq(dY)[L,N] . deq(W)[N,K]   (src/Metis/Metis/bitlinear.py:507-508)
 *   dy_* : dY packed with blocks along N (metis_nvfp4_quant_sr_row of dY [L,N])
 *   wt_* : W packed with blocks along N  (metis_nvfp4_quant_col of W [N,K] -> [K, N/2])
 */
int metis_linear_dgrad(const void *dy_codes, const void *dy_scales, const float *dy_unit,
                       const void *wt_codes, const void *wt_scales, const float *wt_unit, int64_t L,
                       int64_t N, int64_t K, void *grad_input, int out_dtype, void *stream);

/*
 * grad_weight[N,K] = deq(dY)^T[N,L] . deq(X)[L,K]  in binary32 (src/Metis/Metis/bitlinear.py:502-510)
 *   dyt_* : dY packed with blocks along L (metis_nvfp4_quant_sr_col of dY [L,N] -> [N, L/2])
 *   xt_*  : X  packed with blocks along L (metis_nvfp4_quant_sr_col of X  [L,K] -> [K, L/2])
 */
int metis_linear_wgrad(const void *dyt_codes, const void *dyt_scales, const float *dyt_unit,
                       const void *xt_codes, const void *xt_scales, const float *xt_unit, int64_t L,
                       int64_t N, int64_t K, void *grad_weight, int out_dtype, void *stream);

/*
 * The three contractions above with caller-supplied scratch for splitting K.  A shape whose 256 x 256
 * output tiles number at most half the compute units of the device (a few hundred to a few thousand
 * rows against a long contraction: short prefill batches, the down projection, dgrad of a narrow layer)
 * leaves most of the device idle in the plain entry points; here up to 16 workgroups share a tile, each
 * contracts its own range of K into a binary32 partial tile in the workspace, and a second kernel adds
 * the partials in ascending order of K and writes the output.  The order of the binary32 additions
 * differs from the unsplit kernels'; the exact products and the result's tolerance do not.
 *
 * metis_linear_workspace_bytes(M, N, K) is what the call needs for an M x N output contracted over K on
 * the CURRENT device (dgrad: L, K, N; wgrad: N, K, L); 0 means the shape is not split and workspace may
 * be NULL.  A workspace that is too small or not 16-byte aligned is METIS_E_WORKSPACE; workspace == NULL
 * always selects the unsplit kernels.  The workspace needs no initialisation and carries nothing
 * between calls; calls that overlap in time need separate workspaces.
 * No counterpart in the reference, whose matmuls go to the vendor library
 * (src/Metis/Metis/bitlinear.py:435-438,502-510).
 */
size_t metis_linear_workspace_bytes(int64_t M, int64_t N, int64_t K);
int metis_linear_fwd_ws(const void *a_codes, const void *a_scales, const float *a_unit,
                        const void *b_codes, const void *b_scales, const float *b_unit, int64_t M,
                        int64_t N, int64_t K, const void *t, const void *u, int64_t r,
                        const void *bias, void *out, int out_dtype, void *workspace,
                        size_t workspace_bytes, void *stream);
int metis_linear_dgrad_ws(const void *dy_codes, const void *dy_scales, const float *dy_unit,
                          const void *wt_codes, const void *wt_scales, const float *wt_unit,
                          int64_t L, int64_t N, int64_t K, void *grad_input, int out_dtype,
                          void *workspace, size_t workspace_bytes, void *stream);
int metis_linear_wgrad_ws(const void *dyt_codes, const void *dyt_scales, const float *dyt_unit,
                          const void *xt_codes, const void *xt_scales, const float *xt_unit,
                          int64_t L, int64_t N, int64_t K, void *grad_weight, int out_dtype,
                          void *workspace, size_t workspace_bytes, void *stream);

/*
 * Rank-r projection of the low-rank branch for decode-sized batches (M < 256):
 *     xv[M, R] = x[M, K] . v[R, K]^T   bf16 operands and result, binary32 accumulation
 *     t [M, R] = bf16(xv * s[R])       when t != NULL
 * `vlinear(x)` and `torch.mul(self.s, y)` of BitLinear.forward with the bf16 V of the north-star formula
 * (src/Metis/Metis/bitlinear.py:752-756).  The contraction is cut into up to 32 chunks that run as separate
 * workgroups (the vendor library walks all of K in one or a few workgroups: 35 us at 64 x 64 x 18944) and a second
 * kernel adds the chunks in order.  Larger batches are served well by the vendor library.
 *   x  bf16 [M, K], row stride ldx (% 8 == 0), 16-byte aligned;  v bf16 [R, K] contiguous;  s bf16 [R]
 *   R % 32 == 0, R <= 256, K % 64 == 0, M < 256 (METIS_E_SHAPE otherwise)
 *   workspace  metis_lowrank_project_workspace_bytes(M, R, K) bytes, 16-byte aligned, no initialisation
 */
size_t metis_lowrank_project_workspace_bytes(int64_t M, int64_t R, int64_t K);
int metis_lowrank_project(const void *x, int64_t ldx, const void *v, int64_t M, int64_t R, int64_t K,
                          const void *s, void *xv, void *t, void *workspace, size_t workspace_bytes,
                          void *stream);

/*
 * The same projection for training and prefill batches (any M; meant for M >= 256), one pass over x:
 *     xv[M, R] = x[M, K] . v[R, K]^T,  t = bf16(xv * s) when t != NULL     (src/Metis/Metis/bitlinear.py:752-756)
 * and, with v = U^T [r, N] and x = dY [L, N], the product dY . U of the backward pass.
 *   R in {32, 64, 128}, K % 64 == 0, ldx % 8 == 0 (METIS_E_SHAPE otherwise); x, v 16-byte aligned; no workspace
 */
int metis_lowrank_project_rows(const void *x, int64_t ldx, const void *v, int64_t M, int64_t R, int64_t K,
                               const void *s, void *xv, void *t, void *stream);

/*
 * metis_lowrank_project_rows with K slices: a tensor of a few thousand rows gives one workgroup of 32 rows per compute
 * unit, too few bytes in flight; with a workspace several workgroups share a row tile, each over its own range of K,
 * and a second small launch adds their binary32 partial sums in slice order (deterministic; the sums are grouped
 * differently from the one-slice call, so the last bit of xv may differ from it).
 *   workspace  metis_lowrank_project_rows_workspace_bytes(M, R, K) bytes (0: one slice is enough), 16-byte aligned;
 *              NULL or a smaller buffer: fewer slices, down to the call above
 */
size_t metis_lowrank_project_rows_workspace_bytes(int64_t M, int64_t R, int64_t K);
int metis_lowrank_project_rows_ws(const void *x, int64_t ldx, const void *v, int64_t M, int64_t R, int64_t K,
                                  const void *s, void *xv, void *t, void *workspace, size_t workspace_bytes,
                                  void *stream);

/*
 * Both things BitLinear.forward does with its activation, in one pass over it: the NVFP4 quantization that feeds the
 * residual branch (src/Metis/Metis/bitlinear.py:566-576 via quant.py:6-36) and the rank-r projection of the low-rank
 * branch (bitlinear.py:752-756).  Results: xv / t as metis_lowrank_project_rows_ws, codes / deferred as
 * metis_nvfp4_quant_row_deferred (same bytes), i.e. round to nearest, rows, scale bytes left to the consumer
 * (metis_nvfp4_expand_tiled_deferred, metis_nvfp4_deferred_scales).
 *   x  bf16 [rows, cols] contiguous, 16-byte aligned; cols % 64 == 0; R in {32, 64}; rows <= 65536
 *      (METIS_E_TOO_LARGE beyond: call the two functions separately)
 *   mode  METIS_MODE_P32 or METIS_MODE_PB16 (arithmetic of the quantizer; the projection is bf16 x bf16 -> binary32)
 */
int metis_nvfp4_quant_project_deferred(const void *x, int64_t rows, int64_t cols, int mode, const void *v,
                                       int64_t R, const void *s, void *xv, void *t, void *codes,
                                       void *deferred, size_t deferred_bytes, void *workspace,
                                       size_t workspace_bytes, void *stream);

/*
 * Gradient of the scale vector s of the low-rank branch, y = s * (x V^T) (src/Metis/Metis/bitlinear.py:755):
 *     out[c] = sum_l bf16(g[l, c] * xv[l, c])      g = dY U, xv = x V^T, both bf16 [L, R] contiguous; out [R] of
 *                                                  out_dtype (METIS_DTYPE_F32, or _BF16: the sum rounded once)
 * the product rounded to bf16 as autograd forms it for torch.mul on bf16 tensors, the sum in binary32 in a fixed order.
 * One launch in place of the multiply, fill, reduction and cast that torch runs.  R % 8 == 0 (METIS_E_SHAPE otherwise);
 * g and xv 16-byte aligned; L == 0 writes zeros.
 */
int metis_lowrank_scale_grad(const void *g, const void *xv, int64_t L, int64_t R, void *out, int out_dtype,
                             void *stream);

/*
 * The rank-r products of the backward pass that contract over tokens:
 *     out[C, R] = sum_l a[l, C] * b[l, R]        bf16 operands, binary32 accumulation
 * a = dY [L, N], b = (x V^T) * s  ->  gradient of U [N, r];   a = x [L, K], b = (dY U) * s, transpose = 1  ->
 * gradient of V [r, K].  Replaces the torch matmuls autograd runs for ulinear / vlinear
 * (src/Metis/Metis/bitlinear.py:752-757).  Tokens are cut into slices that run as separate workgroups; their
 * binary32 partial results meet in the workspace and are added in slice order (deterministic).
 *   R in {32, 64, 128}, C % 8 == 0, lda % 8 == 0 (METIS_E_SHAPE otherwise); a, b 16-byte aligned, b contiguous
 *   out       [C, R], or [R, C] when transpose != 0, of out_dtype
 *   workspace metis_lowrank_tokens_workspace_bytes(L, C, R) bytes, 16-byte aligned, no initialisation
 */
size_t metis_lowrank_tokens_workspace_bytes(int64_t L, int64_t C, int64_t R);
int metis_lowrank_contract_tokens(const void *a, int64_t lda, const void *b, int64_t L, int64_t C, int64_t R,
                                  void *out, int out_dtype, int transpose, void *workspace,
                                  size_t workspace_bytes, void *stream);

/*
 * One packed activation against several weight matrices in one call: the q/k/v (gate/up) projections of a
 * decoder layer, which the reference quantizes the activation once for (BitLinear._get_shared_quantized_input,
 * src/Metis/Metis/bitlinear.py:676-702) and then multiplies one by one.  Result i equals
 * metis_linear_fwd(a, members[i].b_*, M, members[i].N, K, members[i].t, .u, .r, .bias, members[i].out).
 * For decode-sized M (< 256, K % 64 == 0, count <= 4) all members share one launch, so a narrow k or v projection
 * no longer costs a launch latency of its own; other shapes run member by member.
 *   members  HOST array of `count` descriptors holding device pointers (bias [N] or NULL)
 */
typedef struct metis_linear_member {
    const void *b_codes, *b_scales;
    const float *b_unit;
    const void *t, *u;
    int64_t r;
    const void *bias;
    void *out;
    int64_t N;
    int64_t bias_is_f32; /* 0: bias is bf16 [N]; 1: binary32 [N] (metis_linear_fwd_f32bias) */
    int64_t ldt;         /* row stride of t in elements; 0 = r.  A stride other than r (members reading their columns of
                            one stacked [M, sum r] projection) needs M < 256 and K % 64 == 0, else METIS_E_ARG */
    const void *b_decode; /* NULL, or the same packed weight in the decode layout (metis_nvfp4_decode_weight; K % 256 == 0,
                            16-byte aligned): the decode-sized kernel then streams it as whole lines and b_codes /
                            b_scales may be NULL.  Calls that do not run on the decode-sized kernel need b_codes / b_scales */
} metis_linear_member;
/* sizeof(metis_linear_member) as the library was built: a caller compiled against another revision of this header
 * compares it with its own before passing member arrays (a mismatch would make the library read past the caller's array). */
size_t metis_linear_member_size(void);
/* A packed weight [N, K] in the decode layout, derived data to be cached beside the packed form (the reference caches
 * its dequantized weight the same way, src/Metis/Metis/bitlinear.py:563-589): 0.5625 B per element as packed, rows
 * grouped in tiles of 32 and K in steps of 256 so that every load instruction of a wave of the decode-sized kernel
 * reads a KiB of consecutive bytes instead of 16 bytes from each of 64 rows.  K % 256 == 0 (METIS_E_SHAPE otherwise).
 *   out   metis_nvfp4_decode_weight_bytes(N, K) bytes, 16-byte aligned */
size_t metis_nvfp4_decode_weight_bytes(int64_t N, int64_t K);
int metis_nvfp4_decode_weight(const void *codes, const void *scales, int64_t N, int64_t K, void *out, void *stream);

/*
 * Decode-sized activations in the decode layout as well.  Against a row-major packed activation, a load instruction of the
 * decode-sized kernel touches 64 different lines (one per activation row), and every workgroup reads the whole
 * activation: the layout above turns that into one KiB of consecutive bytes per instruction (66 instead of 73 us for the
 * four calls of a Qwen2.5-7B layer at 64 tokens).  The quantizer writes it in its second launch, next to the ordinary
 * scale bytes (no additional launch):
 *   metis_nvfp4_quant_row_decode        metis_nvfp4_quant_row of a contiguous bf16 tensor with rows < 256 and
 *                                       cols % 256 == 0 (mode METIS_MODE_P32 or METIS_MODE_PB16), and `decode`
 *                                       (metis_nvfp4_decode_weight_bytes(rows, cols) bytes, 16-byte aligned)
 *   metis_rmsnorm_nvfp4_quant_decode    metis_rmsnorm_nvfp4_quant likewise
 * and metis_linear_fwd_grouped, metis_linear_fwd_grouped_bf16 and metis_linear_fwd_grouped_centered take it in place of
 * the packed activation: pass the buffer as a_codes and NULL as a_scales (M < 256, K % 256 == 0, weight scale bytes
 * 8-byte aligned; METIS_E_ARG otherwise).  Same kernel, same order of operations: the same bits.
 */
int metis_nvfp4_quant_row_decode(const void *x, int64_t rows, int64_t cols, int mode, void *codes,
                                 void *scales, float *unit, void *decode, void *workspace,
                                 size_t workspace_bytes, void *stream);
int metis_rmsnorm_nvfp4_quant_decode(const void *x, const void *gamma, float eps, int64_t rows,
                                     int64_t cols, int mode, void *normed, void *codes, void *scales,
                                     float *unit, void *decode, void *workspace,
                                     size_t workspace_bytes, void *stream);
int metis_linear_fwd_grouped(const void *a_codes, const void *a_scales, const float *a_unit, int64_t M,
                             int64_t K, const metis_linear_member *members, int count, int out_dtype,
                             void *workspace, size_t workspace_bytes, void *stream);
/* The same call for a layer whose arithmetic is bf16 (both operands packed with METIS_MODE_PB16; compute_dtype =
 * bfloat16 as src/grpo/grpo.py:204-205 configures every patched layer): result i follows the reference's all-bf16
 * evaluation of LinearLowbitFunction.forward / BitLinear.forward (src/Metis/Metis/bitlinear.py:435-438, 752-760) the way
 * metis_linear_tiled_fwd does with mode = METIS_MODE_PB16 -- operands are its twice-rounded bf16 dequantized values,
 * the residual product is rounded to bf16, the bias added in bf16, then the low-rank term and the final rounding (a
 * binary32 `out` receives bf16 values).  Decode-sized shapes only (M < 256, K % 64 == 0, N % 4 == 0, r % 32 == 0,
 * count <= 4, the alignments of the call above): METIS_E_ARG otherwise -- larger batches run on
 * metis_linear_tiled_fwd.  Workspace as above. */
int metis_linear_fwd_grouped_bf16(const void *a_codes, const void *a_scales, const float *a_unit, int64_t M,
                                  int64_t K, const metis_linear_member *members, int count, int out_dtype,
                                  void *workspace, size_t workspace_bytes, void *stream);
/* The activation of a decode-sized call as ready 16-bit MFMA operands, built once per activation instead of being
 * expanded from its codes by every workgroup of every projection that reads it (in bf16 arithmetic the expansion is
 * two roundings per element; q/k/v or gate/up share one activation).
 *   metis_nvfp4_decode_operand   mode METIS_MODE_P32: binary16 e2m1 * e4m3 * 2^-8 (exact, the tensor unit stays
 *                                outside); METIS_MODE_PB16: the reference's bf16 dequantized values, and with `center`
 *                                (bf16 [cols], 16-byte aligned, or NULL; PB16 only) the mean mode's me + QDQ(x - me)
 *                                rounded to bf16 (src/Metis/Metis/bitlinear.py:330-333).  rows < 256, cols % 256 == 0;
 *                                out: metis_nvfp4_decode_operand_bytes(rows, cols) bytes, 16-byte aligned
 *   metis_linear_fwd_grouped_operand  metis_linear_fwd_grouped (mode METIS_MODE_P32, same bits) or
 *                                metis_linear_fwd_grouped_bf16 (mode METIS_MODE_PB16, same bits when no centre went
 *                                into the operand) reading that buffer; a_unit as for the packed activation (unused in
 *                                mode PB16 but required); weight scale pointers 8-byte aligned; METIS_E_ARG for
 *                                shapes the decode-sized kernel does not take
 *   metis_nvfp4_decode_operand_deferred  the same from a tensor whose quantizer call deferred its scale bytes
 *                                (metis_nvfp4_quant_row_deferred: quant_mode = its mode): forms the E4M3 bytes itself and
 *                                writes the tensor unit (float [1], required), so a decode-sized activation costs two
 *                                launches ahead of its GEMMs instead of three
 *   metis_decode_prepare_deferred  metis_lowrank_project (x [rows, cols] bf16 with row stride ldx, v [R, cols], s, xv,
 *                                t, workspace: its arguments and limits) and metis_nvfp4_decode_operand_deferred of
 *                                the same activation (codes, deferred, quant_mode, mode, center, unit, out: its
 *                                arguments and limits) in two launches instead of three: the projection's finishing
 *                                step rides in the first blocks of the operand launch.  Same bits as the two calls
 *                                (`vlinear(x)`, `torch.mul(self.s, y)` and the quantized input of BitLinear.forward,
 *                                src/Metis/Metis/bitlinear.py:752-760).  x = NULL: the workspace already holds the
 *                                projection's partial sums, left there by metis_decode_quant_project_deferred on the
 *                                same rows, cols and R (R <= 128 then): one launch.  rotate != 0: the operand half is
 *                                metis_nvfp4_decode_operand_rht with sign_mask (no centre then; codes 8-byte aligned)
 *   metis_nvfp4_decode_operand_rht  the operand for a call against a weight packed in the ROTATED domain (NV recipe:
 *                                metis_nvfp4_quant_row_rht with sign_mask; the forward multiplies with
 *                                rotate_back(QDQ(rotate(W))), src/Metis/Metis/bitlinear.py:577-585, 395-405).  The
 *                                decode-sized kernel streams that packed weight as it is, so the rotation is applied
 *                                to the activation instead: every dequantized block of 16 rotated forward with the same
 *                                sign_mask and scaled by 1/16 (sums exact, one rounding to the 16-bit operand format),
 *                                which gives the same product.  deferred = NULL: scales / unit as written by the
 *                                quantizer (unit needed in mode PB16 only); otherwise scales is ignored, the parked
 *                                data of metis_nvfp4_quant_row_deferred is read (quant_mode = its mode) and unit
 *                                receives the tensor unit.  Shapes and `out` as metis_nvfp4_decode_operand
 *   metis_decode_quant_project_deferred  metis_nvfp4_quant_row_deferred (no centre; x contiguous bf16 [rows, cols],
 *                                rows < 256, cols % 64 == 0) and, in the same launch, the first step of
 *                                metis_lowrank_project on v [R, cols] (R % 32 == 0, R <= 128; METIS_E_SHAPE otherwise):
 *                                its partial sums go to `workspace` (metis_lowrank_project_workspace_bytes(rows, R,
 *                                cols) bytes, 16-byte aligned) and wait there for metis_decode_prepare_deferred with
 *                                x = NULL.  Same bits as the separate calls: a decode-sized BitLinear.forward is then
 *                                three launches (this, the prepare call, the GEMM) instead of five */
size_t metis_nvfp4_decode_operand_bytes(int64_t rows, int64_t cols);
int metis_nvfp4_decode_operand(const void *codes, const void *scales, const float *unit, int64_t rows,
                               int64_t cols, int mode, const void *center, void *out, void *stream);
int metis_nvfp4_decode_operand_deferred(const void *codes, const void *deferred, int64_t rows, int64_t cols,
                                        int quant_mode, int mode, const void *center, float *unit, void *out,
                                        void *stream);
int metis_nvfp4_decode_operand_rht(const void *codes, const void *scales, float *unit, const void *deferred,
                                   int64_t rows, int64_t cols, int quant_mode, int mode, uint32_t sign_mask,
                                   void *out, void *stream);
int metis_decode_quant_project_deferred(const void *x, int64_t rows, int64_t cols, int mode, void *codes,
                                        void *deferred, size_t deferred_bytes, const void *v, int64_t R,
                                        void *workspace, size_t workspace_bytes, void *stream);
int metis_decode_prepare_deferred(const void *x, int64_t ldx, const void *v, int64_t R, const void *s, void *xv,
                                  void *t, void *workspace, size_t workspace_bytes, const void *codes,
                                  const void *deferred, int64_t rows, int64_t cols, int quant_mode, int mode,
                                  const void *center, float *unit, void *out, int rotate, uint32_t sign_mask,
                                  void *stream);
int metis_linear_fwd_grouped_operand(const void *a_operand, const float *a_unit, int64_t M, int64_t K,
                                     const metis_linear_member *members, int count, int out_dtype, int mode,
                                     void *workspace, size_t workspace_bytes, void *stream);
/* Scratch for the calls above: with few output columns and a long K (a down projection at decode size) K is cut
 * into slices that run as separate workgroups, their binary32 partial sums meet in the workspace and a second
 * small kernel adds them in a fixed order.  Only the N fields of the members are read; the figure is an upper
 * bound (the number of slices also depends on pointer alignment, known only at the call).  0 = the shape is not
 * split; workspace = NULL in the call = never split.  16-byte aligned, contents need no initialisation. */
size_t metis_linear_grouped_workspace_bytes(int64_t M, int64_t K, const metis_linear_member *members, int count);
/* Mean mode for decode-sized batches in one pass over the weights (BitLinear.forward under the reference's default
 * arguments, bitlinear.py:311-336 with the running mean of 316-323): the packed activation holds the centred
 * residual R = Q(X - me) and every output row additionally receives W^ me, accumulated in binary32 inside the
 * GEMM kernel from the weight operands it expands anyway (center: binary32 [K], 16-byte aligned):
 *     out_g = R . W^_g^T + 1 (W^_g center)^T + t_g u_g^T + bias_g.
 * Same result as metis_nvfp4_matvec + metis_linear_fwd_f32bias to about 2^-22 of the centre's magnitude (it enters
 * as a pair of binary16 values hi + lo through one more MFMA per step; |center| < 2^20), without reading the
 * packed weights a second time.  Shapes: those for which ..._supported returns 1 (M < 256, K % 256 == 0, at most
 * four members, scale pointers 8-byte aligned, and the K range of a workgroup small enough for its LDS: K <= 8192
 * unsplit, longer with the workspace); METIS_E_ARG otherwise. */
int metis_linear_fwd_grouped_centered(const void *a_codes, const void *a_scales, const float *a_unit, int64_t M,
                                      int64_t K, const metis_linear_member *members, int count, int out_dtype,
                                      const float *center, void *workspace, size_t workspace_bytes, void *stream);
int metis_linear_grouped_centered_supported(int64_t M, int64_t K, const metis_linear_member *members, int count,
                                            int have_workspace);

/*
 * Mean mode: X^ = 1 me^T + QDQ(X - me), the column mean over tokens kept in high precision and only the
 * centred residual quantized (LinearLowbitFunction.svd_quant with metis_mode="mean",
 * src/Metis/Metis/bitlinear.py:311-336; the default of the reference's MetisArgs, src/grpo/grpo.py:66).
 * A matmul with X^ splits into a GEMM on the packed residual and rank-one terms:
 *     X^ W^T = QDQ(X - me) W^T + 1 (W^ me)^T
 * Three entry points provide the pieces.
 *
 * metis_nvfp4_quant_centered: the quantizers above applied to x - center, the subtraction rounded to the
 * dtype of the mode exactly as the reference's `input_flat - me`.
 *   center  one value per column of x: float [cols] in METIS_MODE_P32 / METIS_MODE_P32_F32 (the residual is
 *           then a binary32 value and is encoded by the literal element rule), bf16 [cols] in
 *           METIS_MODE_PB16; 16-byte aligned
 *   sr, col  0/1: stochastic rounding (noise / seed / offset as in metis_nvfp4_quant_sr_row), column-blocked
 *           and transposed output (as metis_nvfp4_quant_col; the centre still belongs to the columns of x)
 */
int metis_nvfp4_quant_centered(const void *x, int64_t rows, int64_t cols, int64_t ld, int mode,
                               const void *center, int sr, int col, const void *noise, uint64_t seed,
                               uint64_t offset, void *codes, void *scales, float *unit,
                               void *workspace, size_t workspace_bytes, void *stream);

/*
 * me[c] = (sum_r x[r, c]) / rows: the column mean over tokens of the mean mode (`input_flat.mean(dim=0)`,
 * src/Metis/Metis/bitlinear.py:326), binary32 accumulation in a fixed order (slabs of rows, then slabs).
 *   x      [rows, cols] of x_dtype (METIS_DTYPE_BF16 / METIS_DTYPE_F32), row stride ld; cols % 4 == 0, ld % 4 == 0
 *   out    [cols] of out_dtype (float for binary32 arithmetic, bf16 for bf16 arithmetic)
 *   workspace  metis_column_mean_workspace_bytes(cols) bytes, 16-byte aligned, no initialisation needed
 */
size_t metis_column_mean_workspace_bytes(int64_t cols);
int metis_column_mean(const void *x, int64_t rows, int64_t cols, int64_t ld, int x_dtype, void *out,
                      int out_dtype, void *workspace, size_t workspace_bytes, void *stream);
/* The column mean followed by the weighted running mean of single-token decode calls
 * (src/Metis/Metis/bitlinear.py:316-323), in the same two launches:
 *     me = (cached * cached_count + mean(x) * rows) / (cached_count + rows),
 * every operation rounded to out_dtype as the reference's tensor expression rounds it (true division).
 *   cached        [cols] of out_dtype: the mean so far, or NULL (then me = mean(x)); may be the same buffer as out
 *   cached_count  rows that went into it (<= 2^24)
 *   out32         optional float [cols]: me once more as binary32 (what metis_linear_fwd_grouped_centered takes) */
int metis_column_mean_running(const void *x, int64_t rows, int64_t cols, int64_t ld, int x_dtype,
                              const void *cached, int64_t cached_count, void *out, float *out32, int out_dtype,
                              void *workspace, size_t workspace_bytes, void *stream);
/* Same reduction without the division: out[c] = sum_r x[r, c], the bias gradient grad_output.sum(dim=(0, 1))
 * of LinearLowbitFunction.backward (src/Metis/Metis/bitlinear.py:455).  Same arguments and workspace. */
int metis_column_sum(const void *x, int64_t rows, int64_t cols, int64_t ld, int x_dtype, void *out,
                     int out_dtype, void *workspace, size_t workspace_bytes, void *stream);

/*
 * y[i] = alpha * sum_k deq(P)[i, k] * v[k] for a packed [rows, cols] tensor P, binary32 accumulation.
 *   v      float [cols], 16-byte aligned, or NULL for all ones (row sums of the dequantized tensor)
 *   out    float [rows] or NULL
 *   split  bf16 matrix with row stride split_ld, or NULL: y[i] is also written as three bf16 terms
 *          hi + mid + lo (exact to binary32 precision) into columns split_col .. split_col + 2 of row i,
 *          the form in which a rank-one term enters the t / u operands of metis_linear_fwd
 * With P a packed weight and v the mean this is W^ me (forward) or W^T^ me_dy (dgrad); with v = NULL and P
 * a column-blocked residual it is the column sum the weight gradient's rank-one terms need.
 */
int metis_nvfp4_matvec(const void *codes, const void *scales, const float *unit, int64_t rows,
                       int64_t cols, const float *v, float alpha, float *out, void *split,
                       int64_t split_ld, int split_col, void *stream);

/* metis_nvfp4_matvec with an affine tail: out[i] = alpha * sum_k deq(P)[i, k] * v[k] + beta * z[i]  (z float [rows]). */
int metis_nvfp4_matvec_affine(const void *codes, const void *scales, const float *unit, int64_t rows,
                              int64_t cols, const float *v, float alpha, const float *z, float beta,
                              float *out, void *stream);

/*
 * Low-rank operands that carry up to two rank-one terms at binary32 precision:
 *     t [n, 32], u [k, 32] (bf16, row stride 32)  with  t u^T = a1 b1^T + a2 b2^T
 * (each factor split into three bf16 terms, the six leading cross products kept; unused columns zero).
 * a1, a2 float [n]; b1, b2 float [k]; a pair may be NULL together.  The weight gradient of the mean mode,
 *     (1 me_dy^T + R_dy)^T (1 me_x^T + R_x) = R_dy^T R_x + (sum_l R_dy) me_x^T + me_dy (sum_l R_x + L me_x)^T,
 * is then one metis_linear_fwd call on the packed residuals with these t and u.
 */
int metis_rank_one_operands(const float *a1, const float *b1, const float *a2, const float *b2,
                            int64_t n, int64_t k, void *t, void *u, void *stream);

/*
 * metis_linear_fwd_ws with a binary32 bias [N]: the place for bias + W^ me, which a bf16 bias would round
 * to 8 bits.  workspace may be NULL (no split-K).
 */
int metis_linear_fwd_f32bias(const void *a_codes, const void *a_scales, const float *a_unit,
                             const void *b_codes, const void *b_scales, const float *b_unit,
                             int64_t M, int64_t N, int64_t K, const void *t, const void *u,
                             int64_t r, const float *bias, void *out, int out_dtype,
                             void *workspace, size_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* METIS_HIP_H */
