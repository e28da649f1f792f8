// Host-side declarations shared by the translation units of libmetis_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>

#include "../../include/metis_hip.h"

namespace metis {

// Caller-supplied scratch, carved as:
//   [0, 16 KiB)        one partial maximum (uint32 bit pattern) per workgroup of phase 1
//   [16 KiB, +65 KiB)  reduction area of the single-launch quantizer (zero when first used)
//   [81 KiB, ..)       one block maximum per block of 16: bf16 for bf16 input, binary32 for binary32 input
struct Workspace {
    uint32_t* gmax;
    uint32_t* sync;
    uint16_t* amax;
};
constexpr size_t kWsGmaxBytes = 4096 * 4;
constexpr size_t kWsSyncBytes = 260 * 256;     // reduction area of the single-launch quantizer: header, 65 tree nodes and 64 result words on lines of their own, 4096 flags (33 KiB used)

inline size_t workspace_bytes(int64_t rows, int64_t cols)
{
    const size_t nblocks = (size_t)((rows * cols + 15) / 16);
    return kWsGmaxBytes + kWsSyncBytes + ((nblocks * 4 + 255) / 256) * 256;
}

inline int carve_workspace(void* p, size_t bytes, int64_t rows, int64_t cols, Workspace* ws)
{
    if (!p || ((uintptr_t)p % 256) || bytes < workspace_bytes(rows, cols)) return METIS_E_WORKSPACE;
    char* c = static_cast<char*>(p);
    ws->gmax = reinterpret_cast<uint32_t*>(c);
    ws->sync = reinterpret_cast<uint32_t*>(c + kWsGmaxBytes);
    ws->amax = reinterpret_cast<uint16_t*>(c + kWsGmaxBytes + kWsSyncBytes);
    return METIS_OK;
}

// compute units of the current device (cached per device ordinal)
int device_cus();

// Measurement switches (kernel variants and shape overrides read from the environment) exist only in a
// -DMETIS_MEASURE build of the library; the shipped library reads no environment variables.
#ifdef METIS_MEASURE
static inline const char* measure_env(const char* name) { return getenv(name); }
static inline int measure_int(const char* name, int dflt) { const char* v = getenv(name); return v ? atoi(v) : dflt; }
#else
static inline const char* measure_env(const char*) { return nullptr; }
static inline int measure_int(const char*, int dflt) { return dflt; }
#endif

// phase 2 of the quantizer (tensor unit + E4M3 bytes from parked block maxima); nvfp4_quant.hip
// bytes of one block of the decode layout (32 rows x 256 elements of K: four KiB of codes, 512 scale bytes), see gemm_common.h
constexpr int kDecodeBlock = 4096 + 512;
// phase 2 of a quantizer call on a decode-sized tensor (rows < 256, cols % 256 == 0, bf16 block maxima parked): scale bytes
// and unit as launch_scales writes them, and the packed tensor in the decode layout; nvfp4_quant.hip
int launch_scales_decode(int mode, const Workspace& ws, uint32_t ngroups, const void* codes, void* scales, float* unit, int64_t rows,
                         int64_t cols, void* decode, hipStream_t st);
int launch_scales(int mode, const Workspace& ws, uint32_t ngroups, void* scales, float* unit, uint32_t nblocks,
                  hipStream_t st, const void* amax2 = nullptr, void* scales2 = nullptr, float* unit2 = nullptr);

int quantize(const void* x, int64_t rows, int64_t cols, int64_t ld, int mode, bool sr, bool col, const void* noise,
             uint64_t seed, uint64_t offset, void* codes, void* scales, float* unit, void* workspace,
             size_t workspace_bytes, hipStream_t st, const void* center = nullptr, bool resident = false,
             uint32_t spin_limit = 0, void* decode = nullptr);
// both packings (blocks along rows, blocks down columns) of one tensor with stochastic rounding in one pass; nvfp4_quant.hip
int quantize_both_sr(const void* x, int64_t rows, int64_t cols, int64_t ld, int mode, uint64_t seed, uint64_t offset_row,
                     uint64_t offset_col, void* codes_row, void* scales_row, float* unit_row, void* codes_col, void* scales_col,
                     float* unit_col, void* workspace, size_t bytes, hipStream_t st);
// deferred scale bytes (nvfp4_quant.hip): phase 1 alone into caller-owned parked data, phase 2 on it later or never
size_t deferred_bytes(int64_t rows, int64_t cols);
int carve_deferred(void* p, size_t bytes, int64_t rows, int64_t cols, Workspace* ws);
int deferred_grid(uint32_t work_items, int per_cu = 8);
int quantize_row_deferred(const void* x, int64_t rows, int64_t cols, int mode, const void* center, void* codes, void* deferred,
                          size_t bytes, hipStream_t st);
int deferred_scales(const void* deferred, int64_t rows, int64_t cols, int mode, void* scales, float* unit, hipStream_t st);
// the row quantizer on the library's own static scratch (no workspace argument); nvfp4_quant.hip
int quantize_row_static(const void* x, int64_t rows, int64_t cols, int64_t ld, int mode, void* codes, void* scales,
                        float* unit, hipStream_t st);
// codes, scale bytes, unit and the dequantized bf16 tensor of contiguous bf16 rows from one call (two launches); nvfp4_quant.hip
int quantize_lowrank_residual(const void* x, bool x_f32, const void* us, const void* vt, int64_t rows, int64_t cols, int rank, int mode,
                              void* codes, void* scales, float* unit, void* dense, void* workspace, size_t workspace_bytes,
                              hipStream_t st);
int quantize_dequantize_row(const void* x, int64_t rows, int64_t cols, int mode, void* codes, void* scales, float* unit, void* out,
                            void* workspace, size_t workspace_bytes, hipStream_t st);
int dequantize(const void* codes, const void* scales, const float* unit, int64_t rows, int64_t cols, int mode, void* out,
               int out_dtype, hipStream_t st);
int block_scalars(const void* x, int64_t rows, int64_t cols, int mode, void* s, hipStream_t st);
int quant_values(const void* x, const void* s, int64_t rows, int64_t cols, int mode, int sr, const void* noise,
                 uint64_t seed, uint64_t offset, void* out, hipStream_t st);
int rquant_values(const void* xq, void* s, int64_t rows, int64_t cols, int mode, void* out, float* scratch,
                  hipStream_t st);
int rmsnorm_quantize(const void* x, const void* gamma, float eps, int64_t rows, int64_t cols, int mode, void* normed,
                     void* codes, void* scales, float* unit, void* workspace, size_t workspace_bytes, hipStream_t st,
                     bool deferred = false, void* decode = nullptr);
// RMSNorm that also leaves the column mean of its output (mean mode); rmsnorm_quant.hip
size_t rmsnorm_colmean_workspace_bytes(int64_t rows, int64_t cols);
int rmsnorm_colmean(const void* x, const void* gamma, float eps, int64_t rows, int64_t cols, void* normed, void* mean, int mean_bf16,
                    const void* cached, int64_t cached_count, float* mean32, void* workspace, size_t workspace_bytes, hipStream_t st);
int gemm_nvfp4(const void* a_codes, const void* a_scales, const float* a_unit, const void* b_codes, const void* b_scales,
               const float* b_unit, int64_t M, int64_t N, int64_t K, const void* t, const void* u, int64_t r,
               const void* bias, void* out, int out_dtype, hipStream_t st, void* workspace = nullptr,
               size_t workspace_bytes = 0, int bias_f32 = 0);
// y = alpha * unit * deq(codes, scales) . v  (v == NULL: all ones); nvfp4_gemv.hip
int packed_gemv(const void* codes, const void* scales, const float* unit, int64_t rows, int64_t cols, const float* v,
                float alpha, float* out32, void* split, int64_t split_ld, int split_col, hipStream_t st,
                const float* z = nullptr, float beta = 0.0f);
// T [n, 32], U [k, 32] (bf16) with T U^T = a1 b1^T + a2 b2^T to binary32 precision; nvfp4_gemv.hip
int rank_one_operands(const float* a1, const float* b1, const float* a2, const float* b2, int64_t n, int64_t k, void* T, void* U,
                      hipStream_t st);
// one weight matrix of a grouped GEMM (layout shared with metis_linear_member of the C ABI)
struct GemmMember {
    const void* b_codes;
    const void* b_scales;
    const float* b_unit;
    const void* t;
    const void* u;
    int64_t r;
    const void* bias;
    void* out;
    int64_t N;
    int64_t bias_is_f32;
    int64_t ldt;
    const void* b_decode;        // the weight in the decode layout (decode_weight), or nullptr
};
// a packed weight [N, K], K % 256 == 0, in the layout the decode-sized kernel streams as whole lines; metis_gemm.hip
size_t decode_weight_bytes(int64_t N, int64_t K);
int decode_weight(const void* codes, const void* scales, int64_t N, int64_t K, void* out, hipStream_t st);
int gemm_nvfp4_grouped(const void* a_codes, const void* a_scales, const float* a_unit, int64_t M, int64_t K,
                       const GemmMember* members, int count, int out_dtype, hipStream_t st, void* workspace = nullptr,
                       size_t workspace_bytes = 0, const float* center = nullptr, bool pb16 = false, bool a_dense = false);
// the activation of a decode-sized call as ready 16-bit MFMA operands (a_dense above: a_codes is this buffer); metis_gemm.hip
size_t skinny_operand_bytes(int64_t M, int64_t K);
int skinny_operand(const void* codes, const void* scales, const float* unit, int64_t M, int64_t K, int mode, const void* center,
                   void* out, hipStream_t st);
// the same from a tensor whose quantizer call deferred its scale bytes; writes the unit
int skinny_operand_deferred(const void* codes, const void* deferred, int64_t M, int64_t K, int qmode, int mode, const void* center,
                            float* unit_out, void* out, hipStream_t st);
// the same operand for a call against a ROTATED packed weight (NV recipe): activation blocks rotated forward / 16
int skinny_operand_rht(const void* codes, const void* scales, float* unit, const void* deferred, int64_t M, int64_t K, int qmode, int mode,
                       uint32_t sign_mask, void* out, hipStream_t st);
// quantize_row_deferred of a decode-sized activation with the projection's first step in the same launch; nvfp4_quant.hip
int quantize_row_deferred_partial(const void* x, int64_t rows, int64_t cols, int mode, void* codes, void* deferred, size_t bytes,
                                  const void* v, int64_t R, void* lr_workspace, size_t lr_workspace_bytes, hipStream_t st);
// the decode-sized rank-r projection (lowrank_small) and skinny_operand_deferred of the same activation, the
// projection's finishing step inside the operand launch
int decode_prepare_deferred(const void* x, int64_t ldx, const void* v, int64_t R, const void* s, void* xv, void* t, void* workspace,
                            size_t workspace_bytes, const void* codes, const void* deferred, int64_t M, int64_t K, int qmode, int mode,
                            const void* center, float* unit_out, void* out, hipStream_t st, int rotate = 0, uint32_t sign_mask = 0);
int gemm_grouped_center_supported(int64_t M, int64_t K, const GemmMember* members, int count, int have_workspace);
// bytes of split-K scratch a grouped call can use (only the N fields of the members are read; 0: it would not split)
size_t gemm_grouped_workspace_bytes(int64_t M, int64_t K, const GemmMember* members, int count);
// bytes of split-K scratch gemm_nvfp4 can use for this shape on the current device (0: it would not split)
size_t gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);

// NV recipe (nvfp4_quant.hip): rotate tiles of 16 along the last dimension and quantize the rotated tensor; the rotation alone
int quantize_rht(const void* x, int64_t rows, int64_t cols, int64_t ld, int mode, uint32_t sign_mask, bool sr, uint64_t seed,
                 uint64_t offset, void* codes, void* scales, float* unit, void* workspace, size_t workspace_bytes, hipStream_t st);
int hadamard16(const void* x, int64_t rows, int64_t cols, int64_t ldx, int dtype, int inverse, uint32_t sign_mask, void* out,
               int64_t ldo, hipStream_t st);

// me[c] = mean over rows of x[:, c] (binary32 accumulation); nvfp4_gemv.hip
size_t column_mean_workspace_bytes(int64_t cols);
int column_mean(const void* x, int64_t rows, int64_t cols, int64_t ld, int in_f32, void* out, int out_bf16, void* workspace,
                size_t workspace_bytes, hipStream_t st, bool sum_only = false, const void* cached = nullptr,
                int64_t cached_count = 0, float* out32 = nullptr);

// xv[M, R] = x[M, K] . v[R, K]^T (bf16, binary32 accumulation) and t = bf16(xv * s) for M < 256; lowrank_small.hip
size_t lowrank_small_workspace_bytes(int64_t M, int64_t R, int64_t K);
int lowrank_small(const void* x, int64_t ldx, const void* v, int64_t M, int64_t R, int64_t K, const void* s, void* xv, void* t,
                  void* workspace, size_t workspace_bytes, hipStream_t st);

// the same in two steps, for a caller whose next launch carries the finishing step in its first
// lowrank_small_finish_blocks(M, R) blocks (lowrank_small_steps.h)
int lowrank_small_partial(const void* x, int64_t ldx, const void* v, int64_t M, int64_t R, int64_t K, const void* s, void* xv, void* t,
                          void* workspace, size_t workspace_bytes, hipStream_t st, int* chunks_out);
inline int lowrank_small_finish_blocks(int64_t M, int64_t R) { return (int)((M * R / 4 + 63) / 64); }

// gradient of the rank-r scale vector: column sums of the bf16 products of two [L, R] tensors; lowrank_small.hip
int scale_grad(const void* g, const void* xv, int64_t L, int64_t R, void* out, int out_dtype, hipStream_t st);

// rank-r products at training sizes (bf16, MFMA, one pass over the tall operand); lowrank_large.hip
// workspace (optional): K slices for more workgroups; qmode >= 0: x is quantized in the same pass (deferred scale bytes)
int lowrank_nt(const void* x, int64_t ldx, const void* v, int64_t M, int64_t R, int64_t K, const void* s, void* xv, void* t,
               hipStream_t st, void* workspace = nullptr, size_t workspace_bytes = 0, int qmode = -1, void* codes = nullptr,
               void* deferred = nullptr, size_t deferred_size = 0);
size_t lowrank_nt_workspace_bytes(int64_t M, int64_t R, int64_t K);
size_t lowrank_tn_workspace_bytes(int64_t L, int64_t C, int64_t R);
int lowrank_tn(const void* a, int64_t lda, const void* b, int64_t L, int64_t C, int64_t R, void* out, int out_dtype, int transpose,
               void* workspace, size_t workspace_bytes, hipStream_t st);

int expand_f16(const void* codes, const void* scales, int64_t rows, int64_t cols, void* out, hipStream_t st);
int gemm_expanded(const void* a_exp, const float* a_unit, const void* b_exp, const float* b_unit, int64_t M, int64_t N,
                  int64_t K, const void* t, const void* u, int64_t r, const void* bias, void* out, int out_dtype,
                  hipStream_t st);

// tiled 16-bit expansion of a packed tensor and the pipelined GEMM that consumes it; metis_gemm_pipe.hip
size_t expand_xt_bytes(int64_t rows, int64_t cols);
int expand_xt(const void* codes, const void* scales, const float* unit, int64_t rows, int64_t cols, int mode, void* out,
              hipStream_t st, int rht = 0, uint32_t sign_mask = 0, const void* center = nullptr);
// the same from a tensor whose quantizer call deferred its scale bytes (qmode: the arithmetic it was quantized in); writes the unit
int expand_xt_deferred(const void* codes, const void* deferred, int64_t rows, int64_t cols, int qmode, int mode, const void* center,
                       float* unit_out, void* out, hipStream_t st);
// a dense bf16 / binary32 tensor in the tiled layout (optional per-column bf16 scale first)
int dense_xt(const void* x, int64_t rows, int64_t cols, int64_t ld, int dtype, const void* col_scale, int mode, void* out, hipStream_t st);
// the tiled operand [cols, rows] (contraction over the packed tensor's rows); rows % 32 == 0
int expand_xt_transposed(const void* codes, const void* scales, const float* unit, int64_t rows, int64_t cols, int mode, void* out,
                         hipStream_t st, int rht, uint32_t sign_mask);
size_t gemm_xt_workspace_bytes(int64_t M, int64_t N, int64_t K, int mode);
int gemm_xt(const void* a_xt, const float* a_unit, const void* b_xt, const float* b_unit, int64_t M, int64_t N, int64_t K,
            const void* t, const void* u, int64_t r, const void* bias, int bias_f32, void* out, int out_dtype, int mode,
            void* workspace, size_t workspace_bytes, hipStream_t st);

}  // namespace metis
