// extern "C" surface of libmetis_hip.so (declared in include/metis_hip.h).
#include "metis_host.h"

namespace metis {
int device_cus()
{
    static int cached[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}
}  // namespace metis

using namespace metis;

extern "C" {

int metis_version(void) { return (0 << 16) | (1 << 8) | 0; }

const char* metis_error_string(int code)
{
    switch (code) {
        case METIS_OK: return "ok";
        case METIS_E_ARG: return "invalid argument (null/misaligned pointer, negative size, unknown mode or dtype)";
        case METIS_E_SHAPE: return "NVFP4 block shape (1, 16) does not divide the blocked dimension";
        case METIS_E_WORKSPACE: return "workspace missing, misaligned or too small";
        case METIS_E_LAUNCH: return "HIP runtime rejected a kernel launch";
        case METIS_E_DEVICE: return "unsupported device";
        case METIS_E_TOO_LARGE: return "tensor exceeds the capacity of the library's static scratch (2^26 elements)";
        default: return "unknown error code";
    }
}

size_t metis_nvfp4_workspace_bytes(int64_t rows, int64_t cols)
{
    if (rows < 0 || cols < 0) return 0;
    return workspace_bytes(rows, cols);
}

int metis_nvfp4_quant_row(const void* x, int64_t rows, int64_t cols, int64_t ld, int mode, void* codes, void* scales,
                          float* unit, void* workspace, size_t workspace_bytes, void* stream)
{
    return quantize(x, rows, cols, ld, mode, false, false, nullptr, 0, 0, codes, scales, unit, workspace,
                    workspace_bytes, (hipStream_t)stream);
}

int metis_nvfp4_quant_row_decode(const void* x, int64_t rows, int64_t cols, int mode, void* codes, void* scales, float* unit,
                                 void* decode, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!decode) return METIS_E_ARG;
    return quantize(x, rows, cols, cols, mode, false, false, nullptr, 0, 0, codes, scales, unit, workspace, workspace_bytes,
                    (hipStream_t)stream, nullptr, false, 0, decode);
}

int metis_rmsnorm_nvfp4_quant_decode(const void* x, const void* gamma, float eps, int64_t rows, int64_t cols, int mode, void* normed,
                                     void* codes, void* scales, float* unit, void* decode, void* workspace, size_t workspace_bytes,
                                     void* stream)
{
    if (!decode) return METIS_E_ARG;
    return rmsnorm_quantize(x, gamma, eps, rows, cols, mode, normed, codes, scales, unit, workspace, workspace_bytes,
                            (hipStream_t)stream, false, decode);
}

size_t metis_linear_member_size(void) { return sizeof(metis_linear_member); }

size_t metis_nvfp4_decode_weight_bytes(int64_t N, int64_t K) { return decode_weight_bytes(N, K); }

int metis_nvfp4_decode_weight(const void* codes, const void* scales, int64_t N, int64_t K, void* out, void* stream)
{
    return decode_weight(codes, scales, N, K, out, (hipStream_t)stream);
}

size_t metis_rmsnorm_colmean_workspace_bytes(int64_t rows, int64_t cols) { return rmsnorm_colmean_workspace_bytes(rows, cols); }

int metis_rmsnorm_colmean(const void* x, const void* gamma, float eps, int64_t rows, int64_t cols, void* normed, void* mean, int mean_dtype,
                          const void* cached, int64_t cached_count, float* mean32, void* workspace, size_t workspace_bytes, void* stream)
{
    if (mean_dtype != METIS_DTYPE_BF16 && mean_dtype != METIS_DTYPE_F32) return METIS_E_ARG;
    return rmsnorm_colmean(x, gamma, eps, rows, cols, normed, mean, mean_dtype == METIS_DTYPE_BF16, cached, cached_count, mean32, workspace,
                           workspace_bytes, (hipStream_t)stream);
}

int metis_nvfp4_quant_dequant_row(const void* x, int64_t rows, int64_t cols, int mode, void* codes, void* scales, float* unit,
                                  void* out, void* workspace, size_t workspace_bytes, void* stream)
{
    return quantize_dequantize_row(x, rows, cols, mode, codes, scales, unit, out, workspace, workspace_bytes, (hipStream_t)stream);
}

int metis_nvfp4_quant_row_static(const void* x, int64_t rows, int64_t cols, int64_t ld, int mode, void* codes, void* scales,
                                 float* unit, void* stream)
{
    return quantize_row_static(x, rows, cols, ld, mode, codes, scales, unit, (hipStream_t)stream);
}

int metis_nvfp4_quant_row_resident(const void* x, int64_t rows, int64_t cols, int mode, void* codes, void* scales,
                                   float* unit, void* workspace, size_t workspace_bytes, uint32_t spin_limit, void* stream)
{
    return quantize(x, rows, cols, cols, mode, false, false, nullptr, 0, 0, codes, scales, unit, workspace,
                    workspace_bytes, (hipStream_t)stream, nullptr, true, spin_limit);
}

int metis_nvfp4_quant_col(const void* x, int64_t rows, int64_t cols, int64_t ld, int mode, void* codes, void* scales,
                          float* unit, void* workspace, size_t workspace_bytes, void* stream)
{
    return quantize(x, rows, cols, ld, mode, false, true, nullptr, 0, 0, codes, scales, unit, workspace,
                    workspace_bytes, (hipStream_t)stream);
}

int metis_nvfp4_quant_sr_row(const void* x, int64_t rows, int64_t cols, int64_t ld, int mode, const void* noise,
                             uint64_t seed, uint64_t offset, void* codes, void* scales, float* unit, void* workspace,
                             size_t workspace_bytes, void* stream)
{
    return quantize(x, rows, cols, ld, mode, true, false, noise, seed, offset, codes, scales, unit, workspace,
                    workspace_bytes, (hipStream_t)stream);
}

int metis_nvfp4_quant_sr_col(const void* x, int64_t rows, int64_t cols, int64_t ld, int mode, const void* noise,
                             uint64_t seed, uint64_t offset, void* codes, void* scales, float* unit, void* workspace,
                             size_t workspace_bytes, void* stream)
{
    return quantize(x, rows, cols, ld, mode, true, true, noise, seed, offset, codes, scales, unit, workspace,
                    workspace_bytes, (hipStream_t)stream);
}

int metis_nvfp4_get_scalar(const void* x, int64_t rows, int64_t cols, int mode, void* s, void* stream)
{
    return block_scalars(x, rows, cols, mode, s, (hipStream_t)stream);
}

int metis_nvfp4_quant_values(const void* x, const void* s, int64_t rows, int64_t cols, int mode, int sr, const void* noise,
                             uint64_t seed, uint64_t offset, void* out, void* stream)
{
    return quant_values(x, s, rows, cols, mode, sr, noise, seed, offset, out, (hipStream_t)stream);
}

int metis_nvfp4_rquant(const void* xq, void* s, int64_t rows, int64_t cols, int mode, void* out, float* scratch,
                       void* stream)
{
    return rquant_values(xq, s, rows, cols, mode, out, scratch, (hipStream_t)stream);
}

int metis_nvfp4_dequant(const void* codes, const void* scales, const float* unit, int64_t rows, int64_t cols, int mode,
                        void* out, int out_dtype, void* stream)
{
    return dequantize(codes, scales, unit, rows, cols, mode, out, out_dtype, (hipStream_t)stream);
}

int metis_rmsnorm_nvfp4_quant(const void* x, const void* gamma, float eps, int64_t rows, int64_t cols, int mode,
                              void* normed, void* codes, void* scales, float* unit, void* workspace,
                              size_t workspace_bytes, void* stream)
{
    return rmsnorm_quantize(x, gamma, eps, rows, cols, mode, normed, codes, scales, unit, workspace, workspace_bytes,
                            (hipStream_t)stream);
}

int metis_linear_fwd(const void* a_codes, const void* a_scales, const float* a_unit, const void* b_codes,
                     const void* b_scales, const float* b_unit, int64_t M, int64_t N, int64_t K, const void* t,
                     const void* u, int64_t r, const void* bias, void* out, int out_dtype, void* stream)
{
    return gemm_nvfp4(a_codes, a_scales, a_unit, b_codes, b_scales, b_unit, M, N, K, t, u, r, bias, out, out_dtype,
                      (hipStream_t)stream);
}

int metis_nvfp4_expand_f16(const void* codes, const void* scales, int64_t rows, int64_t cols, void* out, void* stream)
{
    return expand_f16(codes, scales, rows, cols, out, (hipStream_t)stream);
}

int metis_linear_fwd_expanded(const void* a_exp, const float* a_unit, const void* b_exp, const float* b_unit, int64_t M,
                              int64_t N, int64_t K, const void* t, const void* u, int64_t r, const void* bias, void* out,
                              int out_dtype, void* stream)
{
    return gemm_expanded(a_exp, a_unit, b_exp, b_unit, M, N, K, t, u, r, bias, out, out_dtype, (hipStream_t)stream);
}

size_t metis_nvfp4_expand_tiled_bytes(int64_t rows, int64_t cols) { return expand_xt_bytes(rows, cols); }

int metis_nvfp4_expand_tiled(const void* codes, const void* scales, const float* unit, int64_t rows, int64_t cols, int mode,
                             void* out, void* stream)
{
    return expand_xt(codes, scales, unit, rows, cols, mode, out, (hipStream_t)stream);
}

int metis_nvfp4_expand_tiled_rht(const void* codes, const void* scales, const float* unit, int64_t rows, int64_t cols, int mode,
                                 uint32_t sign_mask, int rotate_back, int transpose, void* out, void* stream)
{
    if (transpose) return expand_xt_transposed(codes, scales, unit, rows, cols, mode, out, (hipStream_t)stream, rotate_back != 0, sign_mask);
    return expand_xt(codes, scales, unit, rows, cols, mode, out, (hipStream_t)stream, rotate_back != 0, sign_mask);
}

int metis_nvfp4_quant_sr_both(const void* x, int64_t rows, int64_t cols, int64_t ld, int mode, uint64_t seed, uint64_t offset_row,
                              uint64_t offset_col, void* codes_row, void* scales_row, float* unit_row, void* codes_col,
                              void* scales_col, float* unit_col, void* workspace, size_t workspace_bytes, void* stream)
{
    return quantize_both_sr(x, rows, cols, ld, mode, seed, offset_row, offset_col, codes_row, scales_row, unit_row, codes_col, scales_col,
                            unit_col, workspace, workspace_bytes, (hipStream_t)stream);
}

size_t metis_nvfp4_deferred_bytes(int64_t rows, int64_t cols) { return deferred_bytes(rows, cols); }

int metis_nvfp4_quant_row_deferred(const void* x, int64_t rows, int64_t cols, int mode, const void* center, void* codes, void* deferred,
                                   size_t deferred_bytes, void* stream)
{
    return quantize_row_deferred(x, rows, cols, mode, center, codes, deferred, deferred_bytes, (hipStream_t)stream);
}

int metis_rmsnorm_nvfp4_quant_deferred(const void* x, const void* gamma, float eps, int64_t rows, int64_t cols, int mode, void* normed,
                                       void* codes, void* deferred, size_t deferred_bytes, void* stream)
{
    return rmsnorm_quantize(x, gamma, eps, rows, cols, mode, normed, codes, nullptr, nullptr, deferred, deferred_bytes, (hipStream_t)stream,
                            true);
}

int metis_nvfp4_deferred_scales(const void* deferred, int64_t rows, int64_t cols, int mode, void* scales, float* unit, void* stream)
{
    return deferred_scales(deferred, rows, cols, mode, scales, unit, (hipStream_t)stream);
}

int metis_nvfp4_expand_tiled_deferred(const void* codes, const void* deferred, int64_t rows, int64_t cols, int quant_mode, int mode,
                                      const void* center, float* unit, void* out, void* stream)
{
    return expand_xt_deferred(codes, deferred, rows, cols, quant_mode, mode, center, unit, out, (hipStream_t)stream);
}

int metis_nvfp4_expand_tiled_centered(const void* codes, const void* scales, const float* unit, int64_t rows, int64_t cols,
                                      const void* center, void* out, void* stream)
{
    if (!center) return METIS_E_ARG;
    return expand_xt(codes, scales, unit, rows, cols, METIS_MODE_PB16, out, (hipStream_t)stream, 0, 0, center);
}

int metis_dense_expand_tiled(const void* x, int64_t rows, int64_t cols, int64_t ld, int dtype, const void* col_scale, int mode, void* out,
                             void* stream)
{
    return dense_xt(x, rows, cols, ld, dtype, col_scale, mode, out, (hipStream_t)stream);
}

int metis_nvfp4_quant_row_rht(const void* x, int64_t rows, int64_t cols, int64_t ld, int mode, uint32_t sign_mask, int sr, uint64_t seed,
                              uint64_t offset, void* codes, void* scales, float* unit, void* workspace, size_t workspace_bytes,
                              void* stream)
{
    return quantize_rht(x, rows, cols, ld, mode, sign_mask, sr != 0, seed, offset, codes, scales, unit, workspace, workspace_bytes,
                        (hipStream_t)stream);
}

int metis_hadamard16(const void* x, int64_t rows, int64_t cols, int64_t ldx, int dtype, int inverse, uint32_t sign_mask, void* out,
                     int64_t ldo, void* stream)
{
    return hadamard16(x, rows, cols, ldx, dtype, inverse, sign_mask, out, ldo, (hipStream_t)stream);
}

size_t metis_linear_tiled_workspace_bytes(int64_t M, int64_t N, int64_t K, int mode) { return gemm_xt_workspace_bytes(M, N, K, mode); }

int metis_linear_fwd_tiled(const void* a_xt, const float* a_unit, const void* b_xt, const float* b_unit, int64_t M, int64_t N,
                           int64_t K, const void* t, const void* u, int64_t r, const void* bias, int bias_is_f32, void* out,
                           int out_dtype, int mode, void* workspace, size_t workspace_bytes, void* stream)
{
    return gemm_xt(a_xt, a_unit, b_xt, b_unit, M, N, K, t, u, r, bias, bias_is_f32 != 0, out, out_dtype, mode, workspace,
                   workspace_bytes, (hipStream_t)stream);
}

int metis_linear_dgrad(const void* dy_codes, const void* dy_scales, const float* dy_unit, const void* wt_codes,
                       const void* wt_scales, const float* wt_unit, int64_t L, int64_t N, int64_t K, void* grad_input,
                       int out_dtype, void* stream)
{
    // grad_input[L,K] = dY[L,N] . W[N,K]: contraction over N, both operands blocked along N
    return gemm_nvfp4(dy_codes, dy_scales, dy_unit, wt_codes, wt_scales, wt_unit, L, K, N, nullptr, nullptr, 0, nullptr,
                      grad_input, out_dtype, (hipStream_t)stream);
}

int metis_linear_wgrad(const void* dyt_codes, const void* dyt_scales, const float* dyt_unit, const void* xt_codes,
                       const void* xt_scales, const float* xt_unit, int64_t L, int64_t N, int64_t K, void* grad_weight,
                       int out_dtype, void* stream)
{
    // grad_weight[N,K] = dY^T[N,L] . X[L,K]: contraction over L, both operands blocked along L
    return gemm_nvfp4(dyt_codes, dyt_scales, dyt_unit, xt_codes, xt_scales, xt_unit, N, K, L, nullptr, nullptr, 0,
                      nullptr, grad_weight, out_dtype, (hipStream_t)stream);
}

int metis_nvfp4_quant_centered(const void* x, int64_t rows, int64_t cols, int64_t ld, int mode, const void* center,
                               int sr, int col, const void* noise, uint64_t seed, uint64_t offset, void* codes,
                               void* scales, float* unit, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!center) return METIS_E_ARG;
    return quantize(x, rows, cols, ld, mode, sr != 0, col != 0, sr ? noise : nullptr, seed, offset, codes, scales, unit,
                    workspace, workspace_bytes, (hipStream_t)stream, center);
}

int metis_nvfp4_quant_lowrank_residual(const void* x, int x_dtype, const void* us, const void* vt, int64_t rows, int64_t cols,
                                       int rank, int mode, void* codes, void* scales, float* unit, void* dense, void* workspace,
                                       size_t workspace_bytes, void* stream)
{
    if (x_dtype != METIS_DTYPE_BF16 && x_dtype != METIS_DTYPE_F32) return METIS_E_ARG;
    return quantize_lowrank_residual(x, x_dtype == METIS_DTYPE_F32, us, vt, rows, cols, rank, mode, codes, scales, unit, dense,
                                     workspace, workspace_bytes, (hipStream_t)stream);
}

size_t metis_column_mean_workspace_bytes(int64_t cols) { return column_mean_workspace_bytes(cols); }

int metis_column_mean(const void* x, int64_t rows, int64_t cols, int64_t ld, int x_dtype, void* out, int out_dtype,
                      void* workspace, size_t workspace_bytes, void* stream)
{
    if ((x_dtype != METIS_DTYPE_BF16 && x_dtype != METIS_DTYPE_F32) || (out_dtype != METIS_DTYPE_BF16 && out_dtype != METIS_DTYPE_F32))
        return METIS_E_ARG;
    return column_mean(x, rows, cols, ld, x_dtype == METIS_DTYPE_F32, out, out_dtype == METIS_DTYPE_BF16, workspace,
                       workspace_bytes, (hipStream_t)stream);
}

int metis_column_mean_running(const void* x, int64_t rows, int64_t cols, int64_t ld, int x_dtype, const void* cached,
                              int64_t cached_count, void* out, float* out32, int out_dtype, void* workspace, size_t workspace_bytes,
                              void* stream)
{
    if ((x_dtype != METIS_DTYPE_BF16 && x_dtype != METIS_DTYPE_F32) || (out_dtype != METIS_DTYPE_BF16 && out_dtype != METIS_DTYPE_F32))
        return METIS_E_ARG;
    return column_mean(x, rows, cols, ld, x_dtype == METIS_DTYPE_F32, out, out_dtype == METIS_DTYPE_BF16, workspace,
                       workspace_bytes, (hipStream_t)stream, false, cached, cached_count, out32);
}

int metis_column_sum(const void* x, int64_t rows, int64_t cols, int64_t ld, int x_dtype, void* out, int out_dtype,
                     void* workspace, size_t workspace_bytes, void* stream)
{
    if ((x_dtype != METIS_DTYPE_BF16 && x_dtype != METIS_DTYPE_F32) || (out_dtype != METIS_DTYPE_BF16 && out_dtype != METIS_DTYPE_F32))
        return METIS_E_ARG;
    return column_mean(x, rows, cols, ld, x_dtype == METIS_DTYPE_F32, out, out_dtype == METIS_DTYPE_BF16, workspace,
                       workspace_bytes, (hipStream_t)stream, true);
}

int metis_nvfp4_matvec(const void* codes, const void* scales, const float* unit, int64_t rows, int64_t cols,
                       const float* v, float alpha, float* out, void* split, int64_t split_ld, int split_col, void* stream)
{
    return packed_gemv(codes, scales, unit, rows, cols, v, alpha, out, split, split_ld, split_col, (hipStream_t)stream);
}

int metis_nvfp4_matvec_affine(const void* codes, const void* scales, const float* unit, int64_t rows, int64_t cols,
                              const float* v, float alpha, const float* z, float beta, float* out, void* stream)
{
    if (!out) return METIS_E_ARG;
    return packed_gemv(codes, scales, unit, rows, cols, v, alpha, out, nullptr, 0, 0, (hipStream_t)stream, z, beta);
}

int metis_rank_one_operands(const float* a1, const float* b1, const float* a2, const float* b2, int64_t n, int64_t k,
                            void* t, void* u, void* stream)
{
    return rank_one_operands(a1, b1, a2, b2, n, k, t, u, (hipStream_t)stream);
}

int metis_linear_fwd_f32bias(const void* a_codes, const void* a_scales, const float* a_unit, const void* b_codes,
                             const void* b_scales, const float* b_unit, int64_t M, int64_t N, int64_t K, const void* t,
                             const void* u, int64_t r, const float* bias, void* out, int out_dtype, void* workspace,
                             size_t workspace_bytes, void* stream)
{
    return gemm_nvfp4(a_codes, a_scales, a_unit, b_codes, b_scales, b_unit, M, N, K, t, u, r, bias, out, out_dtype,
                      (hipStream_t)stream, workspace, workspace_bytes, 1);
}

int metis_linear_fwd_grouped(const void* a_codes, const void* a_scales, const float* a_unit, int64_t M, int64_t K,
                             const metis_linear_member* members, int count, int out_dtype, void* workspace,
                             size_t workspace_bytes, void* stream)
{
    static_assert(sizeof(metis_linear_member) == sizeof(GemmMember), "member layouts must agree");
    return gemm_nvfp4_grouped(a_codes, a_scales, a_unit, M, K, reinterpret_cast<const GemmMember*>(members), count, out_dtype,
                              (hipStream_t)stream, workspace, workspace_bytes);
}

int metis_linear_fwd_grouped_bf16(const void* a_codes, const void* a_scales, const float* a_unit, int64_t M, int64_t K,
                                  const metis_linear_member* members, int count, int out_dtype, void* workspace,
                                  size_t workspace_bytes, void* stream)
{
    return gemm_nvfp4_grouped(a_codes, a_scales, a_unit, M, K, reinterpret_cast<const GemmMember*>(members), count, out_dtype,
                              (hipStream_t)stream, workspace, workspace_bytes, nullptr, true);
}

size_t metis_nvfp4_decode_operand_bytes(int64_t rows, int64_t cols) { return skinny_operand_bytes(rows, cols); }

int metis_nvfp4_decode_operand(const void* codes, const void* scales, const float* unit, int64_t rows, int64_t cols, int mode,
                               const void* center, void* out, void* stream)
{
    return skinny_operand(codes, scales, unit, rows, cols, mode, center, out, (hipStream_t)stream);
}

int metis_nvfp4_decode_operand_deferred(const void* codes, const void* deferred, int64_t rows, int64_t cols, int quant_mode, int mode,
                                        const void* center, float* unit, void* out, void* stream)
{
    return skinny_operand_deferred(codes, deferred, rows, cols, quant_mode, mode, center, unit, out, (hipStream_t)stream);
}

int metis_nvfp4_decode_operand_rht(const void* codes, const void* scales, float* unit, const void* deferred, int64_t rows, int64_t cols,
                                   int quant_mode, int mode, uint32_t sign_mask, void* out, void* stream)
{
    return skinny_operand_rht(codes, scales, unit, deferred, rows, cols, quant_mode, mode, sign_mask, out, (hipStream_t)stream);
}

int metis_decode_quant_project_deferred(const void* x, int64_t rows, int64_t cols, int mode, void* codes, void* deferred,
                                        size_t deferred_bytes, const void* v, int64_t R, void* workspace, size_t workspace_bytes,
                                        void* stream)
{
    return quantize_row_deferred_partial(x, rows, cols, mode, codes, deferred, deferred_bytes, v, R, workspace, workspace_bytes,
                                         (hipStream_t)stream);
}

int metis_decode_prepare_deferred(const void* x, int64_t ldx, const void* v, int64_t R, const void* s, void* xv, void* t,
                                  void* workspace, size_t workspace_bytes, const void* codes, const void* deferred, int64_t rows,
                                  int64_t cols, int quant_mode, int mode, const void* center, float* unit, void* out, int rotate,
                                  uint32_t sign_mask, void* stream)
{
    return decode_prepare_deferred(x, ldx, v, R, s, xv, t, workspace, workspace_bytes, codes, deferred, rows, cols, quant_mode, mode,
                                   center, unit, out, (hipStream_t)stream, rotate, sign_mask);
}

int metis_linear_fwd_grouped_operand(const void* a_operand, const float* a_unit, int64_t M, int64_t K,
                                     const metis_linear_member* members, int count, int out_dtype, int mode, void* workspace,
                                     size_t workspace_bytes, void* stream)
{
    if (mode != METIS_MODE_P32 && mode != METIS_MODE_PB16) return METIS_E_ARG;
    return gemm_nvfp4_grouped(a_operand, nullptr, a_unit, M, K, reinterpret_cast<const GemmMember*>(members), count, out_dtype,
                              (hipStream_t)stream, workspace, workspace_bytes, nullptr, mode == METIS_MODE_PB16, true);
}

int metis_linear_fwd_grouped_centered(const void* a_codes, const void* a_scales, const float* a_unit, int64_t M, int64_t K,
                                      const metis_linear_member* members, int count, int out_dtype, const float* center,
                                      void* workspace, size_t workspace_bytes, void* stream)
{
    if (!center) return METIS_E_ARG;
    return gemm_nvfp4_grouped(a_codes, a_scales, a_unit, M, K, reinterpret_cast<const GemmMember*>(members), count, out_dtype,
                              (hipStream_t)stream, workspace, workspace_bytes, center);
}

int metis_linear_grouped_centered_supported(int64_t M, int64_t K, const metis_linear_member* members, int count, int have_workspace)
{
    return gemm_grouped_center_supported(M, K, reinterpret_cast<const GemmMember*>(members), count, have_workspace);
}

size_t metis_linear_grouped_workspace_bytes(int64_t M, int64_t K, const metis_linear_member* members, int count)
{
    return gemm_grouped_workspace_bytes(M, K, reinterpret_cast<const GemmMember*>(members), count);
}

size_t metis_lowrank_project_workspace_bytes(int64_t M, int64_t R, int64_t K) { return lowrank_small_workspace_bytes(M, R, K); }

int metis_lowrank_project(const void* x, int64_t ldx, const void* v, int64_t M, int64_t R, int64_t K, const void* s, void* xv,
                          void* t, void* workspace, size_t workspace_bytes, void* stream)
{
    return lowrank_small(x, ldx, v, M, R, K, s, xv, t, workspace, workspace_bytes, (hipStream_t)stream);
}

int metis_lowrank_project_rows(const void* x, int64_t ldx, const void* v, int64_t M, int64_t R, int64_t K, const void* s, void* xv,
                               void* t, void* stream)
{
    return lowrank_nt(x, ldx, v, M, R, K, s, xv, t, (hipStream_t)stream);
}

int metis_lowrank_scale_grad(const void* g, const void* xv, int64_t L, int64_t R, void* out, int out_dtype, void* stream)
{
    return scale_grad(g, xv, L, R, out, out_dtype, (hipStream_t)stream);
}

size_t metis_lowrank_project_rows_workspace_bytes(int64_t M, int64_t R, int64_t K) { return lowrank_nt_workspace_bytes(M, R, K); }

int metis_lowrank_project_rows_ws(const void* x, int64_t ldx, const void* v, int64_t M, int64_t R, int64_t K, const void* s, void* xv,
                                  void* t, void* workspace, size_t workspace_bytes, void* stream)
{
    return lowrank_nt(x, ldx, v, M, R, K, s, xv, t, (hipStream_t)stream, workspace, workspace_bytes);
}

int metis_nvfp4_quant_project_deferred(const void* x, int64_t rows, int64_t cols, int mode, const void* v, int64_t R, const void* s,
                                       void* xv, void* t, void* codes, void* deferred, size_t deferred_bytes, void* workspace,
                                       size_t workspace_bytes, void* stream)
{
    if (mode != METIS_MODE_P32 && mode != METIS_MODE_PB16) return METIS_E_ARG;
    return lowrank_nt(x, cols, v, rows, R, cols, s, xv, t, (hipStream_t)stream, workspace, workspace_bytes, mode, codes, deferred,
                      deferred_bytes);
}

size_t metis_lowrank_tokens_workspace_bytes(int64_t L, int64_t C, int64_t R) { return lowrank_tn_workspace_bytes(L, C, R); }

int metis_lowrank_contract_tokens(const void* a, int64_t lda, const void* b, int64_t L, int64_t C, int64_t R, void* out, int out_dtype,
                                  int transpose, void* workspace, size_t workspace_bytes, void* stream)
{
    return lowrank_tn(a, lda, b, L, C, R, out, out_dtype, transpose, workspace, workspace_bytes, (hipStream_t)stream);
}

size_t metis_linear_workspace_bytes(int64_t M, int64_t N, int64_t K) { return gemm_workspace_bytes(M, N, K); }

int metis_linear_fwd_ws(const void* a_codes, const void* a_scales, const float* a_unit, const void* b_codes,
                        const void* b_scales, const float* b_unit, int64_t M, int64_t N, int64_t K, const void* t,
                        const void* u, int64_t r, const void* bias, void* out, int out_dtype, void* workspace,
                        size_t workspace_bytes, void* stream)
{
    return gemm_nvfp4(a_codes, a_scales, a_unit, b_codes, b_scales, b_unit, M, N, K, t, u, r, bias, out, out_dtype,
                      (hipStream_t)stream, workspace, workspace_bytes);
}

int metis_linear_dgrad_ws(const void* dy_codes, const void* dy_scales, const float* dy_unit, const void* wt_codes,
                          const void* wt_scales, const float* wt_unit, int64_t L, int64_t N, int64_t K, void* grad_input,
                          int out_dtype, void* workspace, size_t workspace_bytes, void* stream)
{
    return gemm_nvfp4(dy_codes, dy_scales, dy_unit, wt_codes, wt_scales, wt_unit, L, K, N, nullptr, nullptr, 0, nullptr,
                      grad_input, out_dtype, (hipStream_t)stream, workspace, workspace_bytes);
}

int metis_linear_wgrad_ws(const void* dyt_codes, const void* dyt_scales, const float* dyt_unit, const void* xt_codes,
                          const void* xt_scales, const float* xt_unit, int64_t L, int64_t N, int64_t K, void* grad_weight,
                          int out_dtype, void* workspace, size_t workspace_bytes, void* stream)
{
    return gemm_nvfp4(dyt_codes, dyt_scales, dyt_unit, xt_codes, xt_scales, xt_unit, N, K, L, nullptr, nullptr, 0,
                      nullptr, grad_weight, out_dtype, (hipStream_t)stream, workspace, workspace_bytes);
}

}  // extern "C"
