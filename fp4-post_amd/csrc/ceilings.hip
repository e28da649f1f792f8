// Attainable-ceiling probes for gfx950, loaded by bench.py next to the library (libmetis_ceilings.so): what kernels
// that do nothing but the hot kernels' memory traffic, or nothing but their MFMAs, reach on the device the benchmark
// runs on.  A yardstick beside the published peaks, measured in the same process and at the same clocks as the
// figures it is compared with.  Not part of the product path.
//
//   metis_ceiling_stream   moves the bytes of the NVFP4 quantizer (32 B read, 8 + 2 B written per block of 16) or of
//                          the fused RMSNorm -> NVFP4 (32 B read, 32 + 8 + 2 B written), no arithmetic; whole-line
//                          accesses (a lane owns half a block), the row stores with the non-temporal hint
//   metis_ceiling_mfma     a register-only v_mfma_f32_32x32x16_f16 loop with the GEMM's 4 x 4 tile per wave on operand
//                          fragments read once from a caller buffer (its contents set the switching activity)
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));

template <bool NORMED>
__global__ __launch_bounds__(256) void stream_kernel(const u32x4* __restrict__ x, u32x4* __restrict__ normed, uint32_t* __restrict__ codes,
                                                     uint16_t* __restrict__ amax, uint32_t nchunks)
{
    // a wave owns chunks of 2 KiB (64 blocks): two 16-byte loads per lane, the next chunk in flight
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t step = gridDim.x * 4u;
    uint32_t c = blockIdx.x * 4u + wave;
    u32x4 a = {0, 0, 0, 0}, b = a;
    if (c < nchunks) { a = x[(size_t)c * 128 + lane]; b = x[(size_t)c * 128 + 64 + lane]; }
    while (c < nchunks) {
        const u32x4 ca = a, cb = b;
        const uint32_t n = c + step;
        if (n < nchunks) { a = x[(size_t)n * 128 + lane]; b = x[(size_t)n * 128 + 64 + lane]; }
        if (NORMED) {
            __builtin_nontemporal_store(cb, normed + (size_t)c * 128 + lane);
            __builtin_nontemporal_store(ca, normed + (size_t)c * 128 + 64 + lane);
        }
        codes[(size_t)c * 128 + lane] = ca.x ^ ca.y ^ ca.z ^ ca.w;
        codes[(size_t)c * 128 + 64 + lane] = cb.x ^ cb.y ^ cb.z ^ cb.w;
        amax[(size_t)c * 64 + (lane & 1u) * 32u + (lane >> 1)] = (uint16_t)(ca.x + cb.y);
        c = n;
    }
}

__global__ __launch_bounds__(256) void mfma_kernel(const half8_t* __restrict__ src, float* __restrict__ out, int iters)
{
    half8_t fa[4], fb[4];
    for (int i = 0; i < 4; ++i) {
        fa[i] = src[(threadIdx.x * 8 + i) % 4096];
        fb[i] = src[(threadIdx.x * 8 + 4 + i) % 4096];
    }
    float16_t acc[4][4];
    for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 4; ++j)
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[j], fa[i], acc[i][j], 0, 0, 0);
    }
    float s = 0.0f;
    for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 4; ++j)
            for (int e = 0; e < 16; ++e) s += acc[i][j][e];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

extern "C" {

// elements: a multiple of 1024.  x: 2 B/element; normed: 2 B/element (normed_mix only); codes: 0.5 B/element; amax: 0.125 B/element.
int metis_ceiling_stream(const void* x, void* normed, void* codes, void* amax, int64_t elements, int normed_mix, int grid, void* stream)
{
    if (!x || !codes || !amax || (normed_mix && !normed) || elements <= 0 || elements % 1024 || grid <= 0) return -1;
    const uint32_t nchunks = (uint32_t)(elements / 1024);
    if (normed_mix)
        hipLaunchKernelGGL(stream_kernel<true>, dim3(grid), dim3(256), 0, (hipStream_t)stream, (const u32x4*)x, (u32x4*)normed, (uint32_t*)codes,
                           (uint16_t*)amax, nchunks);
    else
        hipLaunchKernelGGL(stream_kernel<false>, dim3(grid), dim3(256), 0, (hipStream_t)stream, (const u32x4*)x, (u32x4*)normed, (uint32_t*)codes,
                           (uint16_t*)amax, nchunks);
    return hipGetLastError() == hipSuccess ? 0 : -4;
}

// src: 64 KiB of binary16 values; out: grid * 256 floats.  Flops of the launch: grid * 4 waves * iters * 16 MFMAs * 32768.
int metis_ceiling_mfma(const void* src, void* out, int iters, int grid, void* stream)
{
    if (!src || !out || iters <= 0 || grid <= 0) return -1;
    hipLaunchKernelGGL(mfma_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, (const half8_t*)src, (float*)out, iters);
    return hipGetLastError() == hipSuccess ? 0 : -4;
}

}  // extern "C"
