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
#include "lowrank_small_steps.h"
#include "metis_host.h"

namespace metis {

__global__ __launch_bounds__(512) void lowrank_small_partial_kernel(const uint16_t* __restrict__ x, int64_t ldx,
                                                                    const uint16_t* __restrict__ v, int M, int R, int K, int kc,
                                                                    float* __restrict__ ws)
{
    lowrank_small_partial_block((int)blockIdx.x, (int)blockIdx.y, x, ldx, v, M, R, K, kc, ws);
}

__global__ __launch_bounds__(256) void lowrank_small_finish_kernel(const float* __restrict__ ws, int chunks, int MR, int R,
                                                                   const uint16_t* __restrict__ s, uint16_t* __restrict__ xv,
                                                                   uint16_t* __restrict__ t)
{
    lowrank_small_finish_block((int)blockIdx.x, ws, chunks, MR, R, s, xv, t);
}

size_t lowrank_small_workspace_bytes(int64_t M, int64_t R, int64_t K)
{
    if (M <= 0 || R <= 0 || K <= 0) return 0;
    int kc;
    return (size_t)lowrank_small_chunks(K, &kc) * (size_t)M * (size_t)R * sizeof(float);
}

// Argument checks and the first launch (partial sums per K chunk into the workspace); *chunks_out chunks wait for the
// finishing step.  METIS_OK with *chunks_out == 0: nothing to do (M == 0).
int lowrank_small_partial(const void* x, int64_t ldx, const void* v, int64_t M, int64_t R, int64_t K, const void* s, void* xv, void* t,
                          void* workspace, size_t workspace_bytes, hipStream_t st, int* chunks_out)
{
    *chunks_out = 0;
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
    *chunks_out = chunks;
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

int lowrank_small(const void* x, int64_t ldx, const void* v, int64_t M, int64_t R, int64_t K, const void* s, void* xv, void* t,
                  void* workspace, size_t workspace_bytes, hipStream_t st)
{
    int chunks = 0;
    if (const int rc = lowrank_small_partial(x, ldx, v, M, R, K, s, xv, t, workspace, workspace_bytes, st, &chunks)) return rc;
    if (chunks == 0) return METIS_OK;
    const int MR = (int)(M * R);
    hipLaunchKernelGGL(lowrank_small_finish_kernel, dim3((unsigned)lowrank_small_finish_blocks(M, R)), dim3(256), 0, st,
                       (const float*)workspace, chunks, MR, (int)R, (const uint16_t*)s, (uint16_t*)xv, (uint16_t*)t);
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
