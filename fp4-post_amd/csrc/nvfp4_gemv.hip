// Matrix-vector product on a packed NVFP4 matrix:  y[i] = unit * sum_k e2m1(code[i,k]) * e4m3(scale[i,k/16]) * v[k]
//
// The reference's mean mode keeps the column mean of an activation (or gradient) in high precision and
// quantizes only the centred residual: X^ = 1 me^T + QDQ(X - me)  (src/Metis/Metis/bitlinear.py:311-336).
// Its matmuls then split into a GEMM on the packed residual plus rank-one terms
//     X^ W^T = QDQ(X - me) W^T + 1 (W^ me)^T
// and W^ me, like the column sums sum_l QDQ(.)[l, :] that the weight gradient needs (v = NULL: all ones),
// is this product.  HBM-bound on the packed bytes; one wave per matrix row, v comes from L2.
#include "metis_device.h"
#include "metis_host.h"

namespace metis {

typedef float float2_t __attribute__((ext_vector_type(2)));

// out32 (optional): y as binary32.  split (optional): y as three bf16 terms hi + mid + lo (exact to binary32
// precision) in columns split_col .. split_col + 2 of a bf16 matrix with row stride split_ld: the form in which a
// rank-one term enters the low-rank extension of the GEMM.
__global__ __launch_bounds__(256) void packed_gemv_kernel(const uint2* __restrict__ codes, const uint8_t* __restrict__ scales,
                                                          const float* __restrict__ unit, uint32_t rows, uint32_t nblocks_row,
                                                          const float* __restrict__ v, float alpha, float* __restrict__ out32,
                                                          uint16_t* __restrict__ split, int64_t split_ld, int split_col)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t row = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (row >= rows) return;
    const uint2* crow = codes + (size_t)row * nblocks_row;
    const uint8_t* srow = scales + (size_t)row * nblocks_row;
    float acc = 0.0f;
    for (uint32_t b = lane; b < nblocks_row; b += 64u) {
        const uint2 c = crow[b];
        const float sc = __builtin_amdgcn_cvt_f32_fp8((int)srow[b], 0);
        float part = 0.0f;
        if (v) {
            const float4* vp = reinterpret_cast<const float4*>(v + (size_t)b * kBlock);
            const float4 v0 = vp[0], v1 = vp[1], v2 = vp[2], v3 = vp[3];
            const float w[kBlock] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w, v2.x, v2.y, v2.z, v2.w, v3.x, v3.y, v3.z, v3.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float2_t lo = j == 0 ? __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.x, 1.0f, 0)
                                  : j == 1 ? __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.x, 1.0f, 1)
                                  : j == 2 ? __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.x, 1.0f, 2)
                                           : __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.x, 1.0f, 3);
                const float2_t hi = j == 0 ? __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.y, 1.0f, 0)
                                  : j == 1 ? __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.y, 1.0f, 1)
                                  : j == 2 ? __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.y, 1.0f, 2)
                                           : __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.y, 1.0f, 3);
                part = fmaf(lo[0], w[2 * j], part);
                part = fmaf(lo[1], w[2 * j + 1], part);
                part = fmaf(hi[0], w[8 + 2 * j], part);
                part = fmaf(hi[1], w[8 + 2 * j + 1], part);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float2_t lo = j == 0 ? __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.x, 1.0f, 0)
                                  : j == 1 ? __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.x, 1.0f, 1)
                                  : j == 2 ? __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.x, 1.0f, 2)
                                           : __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.x, 1.0f, 3);
                const float2_t hi = j == 0 ? __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.y, 1.0f, 0)
                                  : j == 1 ? __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.y, 1.0f, 1)
                                  : j == 2 ? __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.y, 1.0f, 2)
                                           : __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.y, 1.0f, 3);
                part += (lo[0] + lo[1]) + (hi[0] + hi[1]);      // E2M1 values: exact sums
            }
        }
        acc = fmaf(part, sc, acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) {
        const float y = acc * (*unit) * alpha;
        if (out32) out32[row] = y;
        if (split) {
            uint16_t* d = split + (int64_t)row * split_ld + split_col;
            const uint32_t h = bf16_bits(y);
            const float r1 = y - __uint_as_float(h << 16);
            const uint32_t m = bf16_bits(r1);
            const float r2 = r1 - __uint_as_float(m << 16);
            d[0] = (uint16_t)h;
            d[1] = (uint16_t)m;
            d[2] = (uint16_t)bf16_bits(r2);
        }
    }
}

int packed_gemv(const void* codes, const void* scales, const float* unit, int64_t rows, int64_t cols, const float* v,
                float alpha, float* out32, void* split, int64_t split_ld, int split_col, hipStream_t st)
{
    if (rows < 0 || cols < 0) return METIS_E_ARG;
    if (cols % kBlock) return METIS_E_SHAPE;
    if (rows == 0) return METIS_OK;
    if (!codes || !scales || !unit || (!out32 && !split)) return METIS_E_ARG;
    if (rows > INT32_MAX || cols / kBlock > INT32_MAX) return METIS_E_ARG;
    if (((uintptr_t)codes % 8) || ((uintptr_t)v % 16) || ((uintptr_t)out32 % 4) || ((uintptr_t)split % 2)) return METIS_E_ARG;
    if (split && (split_col < 0 || split_ld < (int64_t)split_col + 3)) return METIS_E_ARG;
    hipLaunchKernelGGL(packed_gemv_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st, (const uint2*)codes,
                       (const uint8_t*)scales, unit, (uint32_t)rows, (uint32_t)(cols / kBlock), v, alpha, out32,
                       (uint16_t*)split, split_ld, split_col);
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

}  // namespace metis
