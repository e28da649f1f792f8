// The two steps of the decode-sized rank-r projection (lowrank_small.hip) as device functions, so that a launch that has
// other small work to do for the same layer call can carry them in some of its blocks: the first step (partial sums of
// xv = x . v^T per K chunk) beside the activation's quantizer (nvfp4_quant.hip), the finishing step (adds the partial
// sums in chunk order, rounds to bf16 and applies s) beside the build of the activation's GEMM operands (metis_gemm.hip).
#pragma once
#include "metis_device.h"

namespace metis {

typedef __bf16 lr_bf16x8_t __attribute__((ext_vector_type(8)));
typedef float lr_float16_t __attribute__((ext_vector_type(16)));

constexpr int kLrMaxChunks = 128;
constexpr int kLrGroup = kLrMaxChunks / 4;     // chunks per thread of the finishing step

// K in chunks of *kc_out elements (a multiple of 64), at most kLrMaxChunks of them
inline int lowrank_small_chunks(int64_t K, int* kc_out)
{
    int64_t kc = 64;
    if ((K + kc - 1) / kc > kLrMaxChunks) kc = ((K + kLrMaxChunks - 1) / kLrMaxChunks + 63) / 64 * 64;
    *kc_out = (int)kc;
    return (int)((K + kc - 1) / kc);
}

// One workgroup of the first step: K chunk `chunk` (kc elements), rows 64 mtile .. ; wave w owns columns 32 w .. of R
// (waves past R / 32 have nothing to do), so the launch needs at least 2 R threads per workgroup.
__device__ __forceinline__ void lowrank_small_partial_block(int chunk, int mtile, const uint16_t* __restrict__ x, int64_t ldx,
                                                            const uint16_t* __restrict__ v, int M, int R, int K, int kc,
                                                            float* __restrict__ ws)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, hi = lane >> 5;
    if (wave * 32 >= R) return;
    const int m0 = mtile * 64;
    const int k0 = chunk * kc, k1 = min(k0 + kc, K);
    const uint16_t* vp = v + (int64_t)min(wave * 32 + (lane & 31), R - 1) * K + hi * 32;
    const uint16_t* xp[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) xp[i] = x + (int64_t)min(m0 + i * 32 + (lane & 31), M - 1) * ldx + hi * 32;
    lr_float16_t acc[2];
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
            const lr_bf16x8_t fv = __builtin_bit_cast(lr_bf16x8_t, rv[q]);
#pragma unroll
            for (int i = 0; i < 2; ++i)
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fv, __builtin_bit_cast(lr_bf16x8_t, rx[i][q]), acc[i], 0, 0, 0);
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

// One block of 256 threads: four threads per output quad (each a quarter of the chunks, folded in order), 64 quads.
// Every thread of the block has to call it (one barrier inside).
__device__ __forceinline__ void lowrank_small_finish_block(int block, const float* __restrict__ ws, int chunks, int MR, int R,
                                                           const uint16_t* __restrict__ s, uint16_t* __restrict__ xv,
                                                           uint16_t* __restrict__ t)
{
    __shared__ float4 fold[3][64];
    const int q = threadIdx.x & 63, g = threadIdx.x >> 6;      // output quad within the block, chunk group
    const int id = (block * 64 + q) * 4;                       // four consecutive elements of [M, R]
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

}  // namespace metis
