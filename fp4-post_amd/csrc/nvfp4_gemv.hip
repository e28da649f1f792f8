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
// A wave owns R consecutive rows and walks the blocks of 16 columns lane by lane; the 16 values of v a lane
// needs for a block are loaded once and used for all R rows (R = 4 for tall matrices: a quarter of the L1 traffic).
__device__ __forceinline__ float block_dot(const uint2 c, const float (&w)[kBlock])
{
    float part = 0.0f;
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
    return part;
}

// R = 0: four rows per WORKGROUP, its four waves interleaved over the blocks (few, long rows).
template <int R>
__global__ __launch_bounds__(256) void packed_gemv_kernel(const uint2* __restrict__ codes, const uint8_t* __restrict__ scales,
                                                          const float* __restrict__ unit, uint32_t rows, uint32_t nblocks_row,
                                                          const float* __restrict__ v, float alpha, float* __restrict__ out32,
                                                          uint16_t* __restrict__ split, int64_t split_ld, int split_col,
                                                          const float* __restrict__ z, float beta)
{
    constexpr int RR = R ? R : 4;                               // rows per wave (R == 0: per workgroup)
    __shared__ float wave_part[4][4];
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t row0 = R ? (blockIdx.x * 4u + wave) * R : blockIdx.x * 4u;
    if (row0 >= rows) return;                                   // uniform per workgroup when R == 0
    float acc[RR];
#pragma unroll
    for (int r = 0; r < RR; ++r) acc[r] = 0.0f;
    for (uint32_t b = R ? lane : threadIdx.x; b < nblocks_row; b += R ? 64u : 256u) {
        float w[kBlock];
        if (v) {
            const float4* vp = reinterpret_cast<const float4*>(v + (size_t)b * kBlock);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float4 f = vp[q];
                w[4 * q] = f.x; w[4 * q + 1] = f.y; w[4 * q + 2] = f.z; w[4 * q + 3] = f.w;
            }
        } else {
#pragma unroll
            for (int j = 0; j < kBlock; ++j) w[j] = 1.0f;
        }
#pragma unroll
        for (int r = 0; r < RR; ++r) {
            const uint32_t row = min(row0 + r, rows - 1);
            const uint2 c = codes[(size_t)row * nblocks_row + b];
            const float sc = __builtin_amdgcn_cvt_f32_fp8((int)scales[(size_t)row * nblocks_row + b], 0);
            acc[r] = fmaf(block_dot(c, w), sc, acc[r]);
        }
    }
#pragma unroll
    for (int r = 0; r < RR; ++r) acc[r] = wave_sum(acc[r]);
    if (R == 0) {                                               // fold the four waves
        if (lane == 0) {
#pragma unroll
            for (int r = 0; r < RR; ++r) wave_part[wave][r] = acc[r];
        }
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int r = 0; r < RR; ++r) acc[r] = (wave_part[0][r] + wave_part[1][r]) + (wave_part[2][r] + wave_part[3][r]);
    }
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < RR; ++r) {
            const uint32_t row = row0 + r;
            if (row >= rows) break;
            float y = acc[r] * (*unit) * alpha;
            if (z) y = fmaf(beta, z[row], y);
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
}

int packed_gemv(const void* codes, const void* scales, const float* unit, int64_t rows, int64_t cols, const float* v,
                float alpha, float* out32, void* split, int64_t split_ld, int split_col, hipStream_t st, const float* z,
                float beta)
{
    if (rows < 0 || cols < 0) return METIS_E_ARG;
    if (cols % kBlock) return METIS_E_SHAPE;
    if (rows == 0) return METIS_OK;
    if (!codes || !scales || !unit || (!out32 && !split)) return METIS_E_ARG;
    if (rows > INT32_MAX || cols / kBlock > INT32_MAX) return METIS_E_ARG;
    if (((uintptr_t)codes % 8) || ((uintptr_t)v % 16) || ((uintptr_t)out32 % 4) || ((uintptr_t)split % 2) || ((uintptr_t)z % 4)) return METIS_E_ARG;
    if (split && (split_col < 0 || split_ld < (int64_t)split_col + 3)) return METIS_E_ARG;
    // four rows per wave once that still leaves every CU a few workgroups
    if (rows >= (int64_t)device_cus() * 64)
        hipLaunchKernelGGL(packed_gemv_kernel<4>, dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, st, (const uint2*)codes,
                           (const uint8_t*)scales, unit, (uint32_t)rows, (uint32_t)(cols / kBlock), v, alpha, out32,
                           (uint16_t*)split, split_ld, split_col, z, beta);
    else if (rows < (int64_t)device_cus() * 16 && cols >= 4096)    // few long rows: a workgroup per row
        hipLaunchKernelGGL(packed_gemv_kernel<0>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st, (const uint2*)codes,
                           (const uint8_t*)scales, unit, (uint32_t)rows, (uint32_t)(cols / kBlock), v, alpha, out32,
                           (uint16_t*)split, split_ld, split_col, z, beta);
    else
        hipLaunchKernelGGL(packed_gemv_kernel<1>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st, (const uint2*)codes,
                           (const uint8_t*)scales, unit, (uint32_t)rows, (uint32_t)(cols / kBlock), v, alpha, out32,
                           (uint16_t*)split, split_ld, split_col, z, beta);
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

// ---------------------------------------------------------------------------------------------
// Rank-one terms for the low-rank extension of the GEMM:  T [n, 32], U [k, 32] (bf16) with
//     T U^T = a1 b1^T + a2 b2^T      to binary32 precision,
// each binary32 factor split into three bf16 terms x = h + m + l and the six leading cross products kept:
// T columns (h, h, h, m, m, l) against U columns (h, m, l, h, m, h) per term; the other 20 columns are zero.
// The weight gradient of the mean mode carries two such terms (bitlinear.py:311-336 applied to both operands).
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ void split3(float x, uint32_t (&p)[3])
{
    p[0] = bf16_bits(x);
    const float r1 = x - __uint_as_float(p[0] << 16);
    p[1] = bf16_bits(r1);
    p[2] = bf16_bits(r1 - __uint_as_float(p[1] << 16));
}

__global__ __launch_bounds__(256) void rank_one_operands_kernel(const float* __restrict__ a1, const float* __restrict__ b1,
                                                                const float* __restrict__ a2, const float* __restrict__ b2,
                                                                uint32_t n, uint32_t k, uint16_t* __restrict__ T,
                                                                uint16_t* __restrict__ U)
{
    const uint32_t row = blockIdx.x * 256u + threadIdx.x;
    for (int side = 0; side < 2; ++side) {
        const uint32_t limit = side ? k : n;
        if (row >= limit) continue;
        uint32_t h[16] = {};                                    // 32 bf16 values, two per word
        const float* src[2] = {side ? b1 : a1, side ? b2 : a2};
#pragma unroll
        for (int term = 0; term < 2; ++term) {
            if (!src[term]) continue;
            uint32_t p[3];
            split3(src[term][row], p);
            // six columns of this term, as three words
            const uint32_t left[3] = {p[0] | (p[0] << 16), p[0] | (p[1] << 16), p[1] | (p[2] << 16)};      // h h | h m | m l
            const uint32_t right[3] = {p[0] | (p[1] << 16), p[2] | (p[0] << 16), p[1] | (p[0] << 16)};     // h m | l h | m h
#pragma unroll
            for (int w = 0; w < 3; ++w) h[term * 3 + w] = side ? right[w] : left[w];
        }
        uint4* dst = reinterpret_cast<uint4*>((side ? U : T) + (size_t)row * 32);
#pragma unroll
        for (int q = 0; q < 4; ++q) dst[q] = make_uint4(h[4 * q], h[4 * q + 1], h[4 * q + 2], h[4 * q + 3]);
    }
}

int rank_one_operands(const float* a1, const float* b1, const float* a2, const float* b2, int64_t n, int64_t k, void* T, void* U,
                      hipStream_t st)
{
    if (n <= 0 || k <= 0 || n > INT32_MAX || k > INT32_MAX) return METIS_E_ARG;
    if (!T || !U || !a1 != !b1 || !a2 != !b2) return METIS_E_ARG;
    if (((uintptr_t)T % 16) || ((uintptr_t)U % 16) || ((uintptr_t)a1 % 4) || ((uintptr_t)b1 % 4) || ((uintptr_t)a2 % 4) ||
        ((uintptr_t)b2 % 4))
        return METIS_E_ARG;
    const int64_t m = n > k ? n : k;
    hipLaunchKernelGGL(rank_one_operands_kernel, dim3((unsigned)((m + 255) / 256)), dim3(256), 0, st, a1, b1, a2, b2, (uint32_t)n,
                       (uint32_t)k, (uint16_t*)T, (uint16_t*)U);
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

// ---------------------------------------------------------------------------------------------
// Column mean over rows (tokens): me[c] = (sum_r x[r, c]) / rows, binary32 accumulation, the `input_flat.mean(dim=0)`
// of the reference's mean mode (src/Metis/Metis/bitlinear.py:326).  HBM-bound: one read of x.
// Phase 1: a workgroup sums a slab of rows for a strip of 256 columns (thread = 4 adjacent columns, the four
// waves take every fourth row) and leaves one partial row in the workspace; phase 2 adds the partial rows in
// a fixed order, divides and rounds to the output dtype.  No atomics: the result does not depend on timing.
// ---------------------------------------------------------------------------------------------
constexpr int kMeanMaxSlabs = 64;

template <bool IN_F32>
__global__ __launch_bounds__(256) void column_sum_kernel(const void* __restrict__ xv, uint32_t rows, uint32_t cols, int64_t ld,
                                                         float* __restrict__ partial, uint32_t rows_per_slab)
{
    __shared__ float4 part[4][64];
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t c = (blockIdx.x * 64u + lane) * 4u;
    const uint32_t r0 = blockIdx.y * rows_per_slab, r1 = min(r0 + rows_per_slab, rows);
    float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (c < cols) {                                            // cols % 4 == 0: a thread's four columns exist together
#pragma unroll 4
        for (uint32_t r = r0 + wave; r < r1; r += 4u) {
            if (IN_F32) {
                const float4 f = *reinterpret_cast<const float4*>(static_cast<const float*>(xv) + (int64_t)r * ld + c);
                acc.x += f.x; acc.y += f.y; acc.z += f.z; acc.w += f.w;
            } else {
                const uint2 w = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(xv) + (int64_t)r * ld + c);
                acc.x += bf16_lo(w.x); acc.y += bf16_hi(w.x); acc.z += bf16_lo(w.y); acc.w += bf16_hi(w.y);
            }
        }
    }
    part[wave][lane] = acc;
    __syncthreads();
    if (wave == 0 && c < cols) {
        const float4 a = part[0][lane], b = part[1][lane], d = part[2][lane], e = part[3][lane];
        *reinterpret_cast<float4*>(partial + (size_t)blockIdx.y * cols + c) =
            make_float4((a.x + b.x) + (d.x + e.x), (a.y + b.y) + (d.y + e.y), (a.z + b.z) + (d.z + e.z), (a.w + b.w) + (d.w + e.w));
    }
}

// cached (optional, same type as out): the weighted running mean of single-token decode calls,
//     me = (cached * cached_count + this_mean * rows) / (cached_count + rows)
// with every operation rounded to the output type as the reference's tensor expression does
// (src/Metis/Metis/bitlinear.py:316-323; true division, as on the CPU).  out32 (optional): the result once more as binary32.
template <bool OUT_BF16>
__global__ __launch_bounds__(64) void column_mean_finish_kernel(const float* __restrict__ partial, uint32_t slabs, uint32_t cols,
                                                                 float count, void* __restrict__ out, const void* __restrict__ cached,
                                                                 float cached_count, float rows_f, float* __restrict__ out32)
{
    const uint32_t c = blockIdx.x * 64u + threadIdx.x;
    if (c >= cols) return;
    // all loads first (independent, at most kMeanMaxSlabs of them), then the additions in slab order
    float v[kMeanMaxSlabs];
#pragma unroll
    for (uint32_t k = 0; k < (uint32_t)kMeanMaxSlabs; ++k) v[k] = k < slabs ? partial[(size_t)k * cols + c] : 0.0f;
    float s = 0.0f;
#pragma unroll
    for (uint32_t k = 0; k < (uint32_t)kMeanMaxSlabs; ++k) s += v[k];
    auto rnd = [](float x) { return OUT_BF16 ? __uint_as_float(bf16_bits(x) << 16) : x; };
    float m = rnd(s / count);
    if (cached) {
        const float cm = OUT_BF16 ? __uint_as_float((uint32_t)static_cast<const uint16_t*>(cached)[c] << 16)
                                  : static_cast<const float*>(cached)[c];
        const float a = rnd(cm * cached_count), b = rnd(m * rows_f);
        m = rnd(rnd(a + b) / (cached_count + rows_f));
    }
    if (OUT_BF16) static_cast<uint16_t*>(out)[c] = (uint16_t)bf16_bits(m);
    else static_cast<float*>(out)[c] = m;
    if (out32) out32[c] = m;
}

size_t column_mean_workspace_bytes(int64_t cols) { return cols > 0 ? (size_t)kMeanMaxSlabs * (size_t)cols * sizeof(float) : 0; }

int column_mean(const void* x, int64_t rows, int64_t cols, int64_t ld, int in_f32, void* out, int out_bf16, void* workspace,
                size_t workspace_bytes, hipStream_t st, bool sum_only, const void* cached, int64_t cached_count, float* out32)
{
    if (cached && (sum_only || cached_count < 0 || cached_count > (1 << 24) || ((uintptr_t)cached % (out_bf16 ? 2 : 4)))) return METIS_E_ARG;
    if ((uintptr_t)out32 % 4) return METIS_E_ARG;
    if (rows <= 0 || cols <= 0 || ld < cols) return METIS_E_ARG;
    if (cols % 4 || ld % 4) return METIS_E_SHAPE;
    if (!x || !out) return METIS_E_ARG;
    if (rows > INT32_MAX || cols > INT32_MAX) return METIS_E_ARG;
    if (((uintptr_t)x % (in_f32 ? 16 : 8)) || ((uintptr_t)out % 4)) return METIS_E_ARG;
    if (!workspace || ((uintptr_t)workspace % 16) || workspace_bytes < column_mean_workspace_bytes(cols)) return METIS_E_WORKSPACE;
    const uint32_t strips = (uint32_t)((cols + 255) / 256);
    // enough workgroups to fill the device about eight times over, at least 16 rows each, at most kMeanMaxSlabs slabs
    int64_t slabs = (8 * (int64_t)device_cus() + strips - 1) / strips;
    if (slabs > (rows + 15) / 16) slabs = (rows + 15) / 16;
    if (slabs > kMeanMaxSlabs) slabs = kMeanMaxSlabs;
    if (slabs < 1) slabs = 1;
    const uint32_t rows_per_slab = (uint32_t)((rows + slabs - 1) / slabs);
    slabs = (rows + rows_per_slab - 1) / rows_per_slab;
    float* partial = static_cast<float*>(workspace);
    const dim3 grid(strips, (unsigned)slabs);
    if (in_f32)
        hipLaunchKernelGGL(column_sum_kernel<true>, grid, dim3(256), 0, st, x, (uint32_t)rows, (uint32_t)cols, ld, partial, rows_per_slab);
    else
        hipLaunchKernelGGL(column_sum_kernel<false>, grid, dim3(256), 0, st, x, (uint32_t)rows, (uint32_t)cols, ld, partial, rows_per_slab);
    const dim3 g2((unsigned)((cols + 63) / 64));
    if (out_bf16)
        hipLaunchKernelGGL(column_mean_finish_kernel<true>, g2, dim3(64), 0, st, partial, (uint32_t)slabs, (uint32_t)cols,
                           sum_only ? 1.0f : (float)rows, out, cached, (float)cached_count, (float)rows, out32);
    else
        hipLaunchKernelGGL(column_mean_finish_kernel<false>, g2, dim3(64), 0, st, partial, (uint32_t)slabs, (uint32_t)cols,
                           sum_only ? 1.0f : (float)rows, out, cached, (float)cached_count, (float)rows, out32);
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

}  // namespace metis
