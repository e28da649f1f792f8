// Rank-r projection for decode-sized batches:  xv[M, R] = x[M, K] . v[R, K]^T  (bf16 operands and result, binary32
// accumulation), t = bf16(xv * s) -- `vlinear(x)` and `torch.mul(self.s, y)` of BitLinear.forward with the bf16 V of
// the north-star formula (src/Metis/Metis/bitlinear.py:752-756), for M < 256.
//
// The output is tiny (M x R) and the contraction long (K up to 18944): the vendor library runs such a product as one
// or a few workgroups walking all of K (35 us at 64 x 64 x 18944).  Here K is cut into up to 128 chunks of one to three
// 64-element steps (the product is latency-bound: a step is one round trip to memory), one workgroup per chunk and
// 64 rows; wave w owns 32 columns of R (R / 32 waves, at most 8); a lane streams 64 contiguous bytes of its row per
// step straight into MFMA operands (both operands with the same mapping, so K may be visited in that permuted order).
// Partial sums go to a caller-supplied workspace [chunks][M][R] and a second small kernel adds them in chunk order
// (four threads per output quad, each a quarter of the chunks, folded in order), rounds to bf16 and applies s.
#include "metis_device.h"
#include "metis_host.h"

namespace metis {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kLrMaxChunks = 128;
constexpr int kLrGroup = kLrMaxChunks / 4;     // chunks per thread of the finish kernel

__global__ __launch_bounds__(512) void lowrank_small_partial_kernel(const uint16_t* __restrict__ x, int64_t ldx,
                                                                    const uint16_t* __restrict__ v, int M, int R, int K, int kc,
                                                                    float* __restrict__ ws)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, hi = lane >> 5;
    if (wave * 32 >= R) return;
    const int chunk = blockIdx.x, m0 = blockIdx.y * 64;
    const int k0 = chunk * kc, k1 = min(k0 + kc, K);
    const uint16_t* vp = v + (int64_t)min(wave * 32 + (lane & 31), R - 1) * K + hi * 32;
    const uint16_t* xp[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) xp[i] = x + (int64_t)min(m0 + i * 32 + (lane & 31), M - 1) * ldx + hi * 32;
    float16_t acc[2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][e] = 0.0f;
    for (int k = k0; k < k1; k += 64) {                        // kc % 64 == 0 and K % 64 == 0
        uint4 rv[4], rx[2][4];
#pragma unroll
        for (int q = 0; q < 4; ++q) rv[q] = reinterpret_cast<const uint4*>(vp + k)[q];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) rx[i][q] = reinterpret_cast<const uint4*>(xp[i] + k)[q];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const bf16x8_t fv = __builtin_bit_cast(bf16x8_t, rv[q]);
#pragma unroll
            for (int i = 0; i < 2; ++i)
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fv, __builtin_bit_cast(bf16x8_t, rx[i][q]), acc[i], 0, 0, 0);
        }
    }
    // acc[i][e] of lane l: row m = m0 + 32 i + l % 32, column r = 32 wave + 8 (e / 4) + 4 (l / 32) + e % 4
    float* wp = ws + (size_t)chunk * M * R;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int m = m0 + i * 32 + (lane & 31);
        if (m >= M) continue;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int r = wave * 32 + 8 * g + 4 * hi;
            if (r < R)                                          // R % 4 == 0
                *reinterpret_cast<float4*>(wp + (size_t)m * R + r) =
                    make_float4(acc[i][4 * g], acc[i][4 * g + 1], acc[i][4 * g + 2], acc[i][4 * g + 3]);
        }
    }
}

__global__ __launch_bounds__(256) void lowrank_small_finish_kernel(const float* __restrict__ ws, int chunks, int MR, int R,
                                                                   const uint16_t* __restrict__ s, uint16_t* __restrict__ xv,
                                                                   uint16_t* __restrict__ t)
{
    __shared__ float4 fold[3][64];
    const int q = threadIdx.x & 63, g = threadIdx.x >> 6;      // output quad within the block, chunk group
    const int id = (blockIdx.x * 64 + q) * 4;                  // four consecutive elements of [M, R]
    const bool live = id < MR;
    const int per = (chunks + 3) / 4, c0 = g * per;            // this thread's chunks: [c0, c0 + per), per <= kLrGroup
    float4 p[kLrGroup];
#pragma unroll
    for (int c = 0; c < kLrGroup; ++c)
        p[c] = (live && c < per && c0 + c < chunks) ? *reinterpret_cast<const float4*>(ws + (size_t)(c0 + c) * MR + id)
                                                    : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    float4 a = p[0];
#pragma unroll
    for (int c = 1; c < kLrGroup; ++c) { a.x += p[c].x; a.y += p[c].y; a.z += p[c].z; a.w += p[c].w; }
    if (g > 0) fold[g - 1][q] = a;
    __syncthreads();
    if (g > 0 || !live) return;
#pragma unroll
    for (int k = 0; k < 3; ++k) { const float4 b = fold[k][q]; a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w; }
    const uint32_t h[4] = {bf16_bits(a.x), bf16_bits(a.y), bf16_bits(a.z), bf16_bits(a.w)};
    *reinterpret_cast<uint2*>(xv + id) = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
    if (t) {
        const int r = id % R;
        uint32_t u[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) u[e] = bf16_bits(__uint_as_float(h[e] << 16) * bf16_lo(s[r + e]));
        *reinterpret_cast<uint2*>(t + id) = make_uint2(u[0] | (u[1] << 16), u[2] | (u[3] << 16));
    }
}

static int lowrank_small_chunks(int64_t K, int* kc_out)
{
    int64_t kc = 64;
    if ((K + kc - 1) / kc > kLrMaxChunks) kc = ((K + kLrMaxChunks - 1) / kLrMaxChunks + 63) / 64 * 64;
    *kc_out = (int)kc;
    return (int)((K + kc - 1) / kc);
}

size_t lowrank_small_workspace_bytes(int64_t M, int64_t R, int64_t K)
{
    if (M <= 0 || R <= 0 || K <= 0) return 0;
    int kc;
    return (size_t)lowrank_small_chunks(K, &kc) * (size_t)M * (size_t)R * sizeof(float);
}

int lowrank_small(const void* x, int64_t ldx, const void* v, int64_t M, int64_t R, int64_t K, const void* s, void* xv, void* t,
                  void* workspace, size_t workspace_bytes, hipStream_t st)
{
    if (M < 0 || R <= 0 || K <= 0 || ldx < K) return METIS_E_ARG;
    if (M >= 256 || R % 32 || R > 256 || K % 64 || ldx % 8) return METIS_E_SHAPE;
    if (M == 0) return METIS_OK;
    if (!x || !v || !xv || (t && !s)) return METIS_E_ARG;
    if (((uintptr_t)x % 16) || ((uintptr_t)v % 16) || ((uintptr_t)xv % 8) || ((uintptr_t)t % 8) || ((uintptr_t)s % 2)) return METIS_E_ARG;
    if (!workspace || ((uintptr_t)workspace % 16) || workspace_bytes < lowrank_small_workspace_bytes(M, R, K)) return METIS_E_WORKSPACE;
    int kc;
    const int chunks = lowrank_small_chunks(K, &kc);
    hipLaunchKernelGGL(lowrank_small_partial_kernel, dim3((unsigned)chunks, (unsigned)((M + 63) / 64)), dim3((unsigned)(2 * R)), 0, st,
                       (const uint16_t*)x, ldx, (const uint16_t*)v, (int)M, (int)R, (int)K, kc, (float*)workspace);
    const int MR = (int)(M * R);
    hipLaunchKernelGGL(lowrank_small_finish_kernel, dim3((unsigned)((MR / 4 + 63) / 64)), dim3(256), 0, st, (const float*)workspace,
                       chunks, MR, (int)R, (const uint16_t*)s, (uint16_t*)xv, (uint16_t*)t);
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

// ---------------------------------------------------------------------------------------------
// Gradient of s in y = s * (x V^T): g_s[c] = sum_l bf16(g[l, c] * xv[l, c]), the product rounded to bf16 as autograd
// forms it for torch.mul on bf16 tensors (src/Metis/Metis/bitlinear.py:755), the sum in binary32.  Two [L, R] bf16
// tensors, a few hundred KB: one workgroup per 8 columns walks all rows (a thread takes every 256th row, 16 bytes of
// each tensor per row), and the 256 per-thread sums of a column are added in thread order -- a fixed order, one launch.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void scale_grad_kernel(const uint16_t* __restrict__ g, const uint16_t* __restrict__ xv, int L, int R,
                                                         void* __restrict__ out, int out_f32)
{
    __shared__ float part[256][9];
    const int c0 = blockIdx.x * 8, tid = threadIdx.x;
    float acc[8] = {};
    for (int l = tid; l < L; l += 256) {
        const uint4 a = *reinterpret_cast<const uint4*>(g + (int64_t)l * R + c0);
        const uint4 b = *reinterpret_cast<const uint4*>(xv + (int64_t)l * R + c0);
        const uint32_t aw[4] = {a.x, a.y, a.z, a.w}, bw[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            acc[2 * j] += rb(bf16_lo(aw[j]) * bf16_lo(bw[j]));
            acc[2 * j + 1] += rb(bf16_hi(aw[j]) * bf16_hi(bw[j]));
        }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) part[tid][j] = acc[j];
    __syncthreads();
    if (tid < 8) {
        float sum = 0.0f;
        for (int t = 0; t < 256; ++t) sum += part[t][tid];
        if (out_f32) static_cast<float*>(out)[c0 + tid] = sum;
        else static_cast<uint16_t*>(out)[c0 + tid] = (uint16_t)bf16_bits(sum);
    }
}

int scale_grad(const void* g, const void* xv, int64_t L, int64_t R, void* out, int out_dtype, hipStream_t st)
{
    if (L < 0 || R <= 0 || (out_dtype != METIS_DTYPE_BF16 && out_dtype != METIS_DTYPE_F32)) return METIS_E_ARG;
    if (R % 8) return METIS_E_SHAPE;
    if (L > INT32_MAX || R > INT32_MAX) return METIS_E_ARG;
    if (!out || ((uintptr_t)out % 4)) return METIS_E_ARG;
    if (L > 0 && (!g || !xv || ((uintptr_t)g % 16) || ((uintptr_t)xv % 16))) return METIS_E_ARG;
    hipLaunchKernelGGL(scale_grad_kernel, dim3((unsigned)(R / 8)), dim3(256), 0, st, (const uint16_t*)g, (const uint16_t*)xv, (int)L, (int)R,
                       out, (int)(out_dtype == METIS_DTYPE_F32));
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

}  // namespace metis
