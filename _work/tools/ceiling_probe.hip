// Attainable-ceiling probes for MI355X (gfx950): what plain kernels with the quantizer's and the
// GEMM's resource pattern reach on this part, as a yardstick next to the published peaks.
//
//   1. streaming kernels with the byte pattern of the NVFP4 quantizer (32 B read, 8 B written per
//      thread) and of the fused RMSNorm->quant (32 B read, 32 + 8 B written), no arithmetic
//   2. hipMemcpy device-to-device
//   3. a register-only v_mfma_f32_32x32x16_f16 loop with a 4x4 tile per wave (the GEMM's shape),
//      constant operands and N(0,1) operands (switching activity limits the clock on this part)
//
// Stand-alone program: prints one line per probe.  Not part of the library.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#define CK(x)                                                                                   \
    do {                                                                                        \
        hipError_t e_ = (x);                                                                    \
        if (e_ != hipSuccess) {                                                                 \
            printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);               \
            return 1;                                                                           \
        }                                                                                       \
    } while (0)

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));

// one 16-element bf16 block per thread per iteration: 32 B in, 8 B out (+ 32 B out when NORMED)
template <bool NORMED>
__global__ __launch_bounds__(256) void stream_kernel(const uint4* __restrict__ x, uint2* __restrict__ codes,
                                                     uint4* __restrict__ normed, uint32_t nblocks)
{
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < nblocks; i += gridDim.x * 256u) {
        const uint4 a = x[2 * (size_t)i], b = x[2 * (size_t)i + 1];
        codes[i] = make_uint2(a.x ^ a.y ^ a.z ^ a.w, b.x ^ b.y ^ b.z ^ b.w);
        if (NORMED) {
            normed[2 * (size_t)i] = b;
            normed[2 * (size_t)i + 1] = a;
        }
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

template <bool NORMED>
static float time_stream(const uint4* x, uint2* codes, uint4* normed, uint32_t nblocks, int grid, int reps)
{
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    for (int i = 0; i < 5; ++i) hipLaunchKernelGGL(stream_kernel<NORMED>, dim3(grid), dim3(256), 0, 0, x, codes, normed, nblocks);
    (void)hipEventRecord(e0);
    for (int i = 0; i < reps; ++i) hipLaunchKernelGGL(stream_kernel<NORMED>, dim3(grid), dim3(256), 0, 0, x, codes, normed, nblocks);
    (void)hipEventRecord(e1);
    (void)hipEventSynchronize(e1);
    float ms = 0.0f;
    (void)hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return ms / reps * 1e3f;
}

int main()
{
    // ---- streaming: config 1 (8192 x 4096) and config 2 (16384 x 4096) element counts
    const size_t elems = (size_t)16384 * 4096;
    uint4 *x, *normed;
    uint2* codes;
    CK(hipMalloc(&x, elems * 2));
    CK(hipMalloc(&normed, elems * 2));
    CK(hipMalloc(&codes, elems / 2));
    CK(hipMemset(x, 1, elems * 2));
    const int grids[] = {1024, 2048, 4096};
    for (int cfg = 0; cfg < 2; ++cfg) {
        const size_t n = cfg == 0 ? elems / 2 : elems;
        const uint32_t nblocks = (uint32_t)(n / 16);
        float best = 1e30f;
        int best_grid = 0;
        for (int g : grids) {
            const float us = cfg == 0 ? time_stream<false>(x, codes, normed, nblocks, g, 50)
                                      : time_stream<true>(x, codes, normed, nblocks, g, 50);
            if (us < best) { best = us; best_grid = g; }
        }
        const double bytes = cfg == 0 ? n * 2.5 : n * 4.5;
        printf("stream %-34s %8.2f us  %6.2f TB/s  (grid %d x 256)\n",
               cfg == 0 ? "quantizer pattern, 33.5 M elements:" : "norm+quant pattern, 67.1 M elements:", best,
               bytes / best / 1e6, best_grid);
    }
    {
        hipEvent_t e0, e1;
        (void)hipEventCreate(&e0);
        (void)hipEventCreate(&e1);
        for (int i = 0; i < 5; ++i) (void)hipMemcpyAsync(normed, x, elems, hipMemcpyDeviceToDevice, 0);
        (void)hipEventRecord(e0);
        for (int i = 0; i < 50; ++i) (void)hipMemcpyAsync(normed, x, elems, hipMemcpyDeviceToDevice, 0);
        (void)hipEventRecord(e1);
        (void)hipEventSynchronize(e1);
        float ms = 0.0f;
        (void)hipEventElapsedTime(&ms, e0, e1);
        printf("hipMemcpy device-to-device, 64 MiB:        %8.2f us  %6.2f TB/s  (read + write)\n", ms / 50 * 1e3,
               2.0 * elems / (ms / 50 * 1e3) / 1e6);
    }

    // ---- MFMA
    float* out;
    half8_t* src;
    CK(hipMalloc(&out, (size_t)512 * 256 * 4));
    CK(hipMalloc(&src, 4096 * 16));
    _Float16* h = (_Float16*)malloc(4096 * 16);
    const int iters = 4000;
    for (int data = 0; data < 2; ++data) {
        srand(1);
        for (int i = 0; i < 4096 * 8; ++i) {
            const float u1 = (float)((rand() + 1.0) / (RAND_MAX + 2.0)), u2 = (float)(rand() / (double)RAND_MAX);
            h[i] = data == 0 ? (_Float16)1.0f : (_Float16)(sqrtf(-2.0f * logf(u1)) * cosf(6.2831853f * u2));
        }
        CK(hipMemcpy(src, h, 4096 * 16, hipMemcpyHostToDevice));
        for (int wg_per_cu = 1; wg_per_cu <= 2; ++wg_per_cu) {
            const int grid = 256 * wg_per_cu;
            hipEvent_t e0, e1;
            (void)hipEventCreate(&e0);
            (void)hipEventCreate(&e1);
            hipLaunchKernelGGL(mfma_kernel, dim3(grid), dim3(256), 0, 0, src, out, iters);
            CK(hipDeviceSynchronize());
            (void)hipEventRecord(e0);
            for (int r = 0; r < 5; ++r) hipLaunchKernelGGL(mfma_kernel, dim3(grid), dim3(256), 0, 0, src, out, iters);
            (void)hipEventRecord(e1);
            (void)hipEventSynchronize(e1);
            float ms = 0.0f;
            (void)hipEventElapsedTime(&ms, e0, e1);
            ms /= 5;
            const double flops = (double)grid * 4 * iters * 16 * 32768.0;
            printf("mfma f16 32x32x16 loop, %-8s operands, %d wave(s)/SIMD: %7.1f TFLOP/s\n", data == 0 ? "constant" : "N(0,1)",
                   wg_per_cu, flops / ms / 1e9);
        }
    }
    free(h);
    return 0;
}
