// The reference's three-call quantizer interface on dequantized tensors, for gfx950:
//   get_scalar(x)   -> raw block scalars [R, C/16]                 (src/Metis/Metis/quant.py:435-455)
//   quant(x, s)     -> E2M1 values {0, +-.5, ..., +-6} as dtype D  (quant.py:459-466 with 118-128 / 137-147)
//   rquant(xq, s)   -> xq * e4m3_roundtrip(s / (max s / 448)) * (max s / 448); s is divided in place
//                                                                   (quant.py:470-548)
// These exist for callers that use the quantizer classes directly (e.g. the SVD-mode activation path,
// src/Metis/Metis/bitlinear.py:283-290); the hot path uses the packed kernels instead.  Literal op
// sequence, element-wise, no attempt at speed.  D = float32 (mode 0) or bf16 (mode 1).
#include "metis_device.h"
#include "metis_host.h"

namespace metis {

template <int MODE> __device__ __forceinline__ float ld(const void* p, int64_t i)
{
    return MODE ? bf16_lo(((const uint16_t*)p)[i]) : ((const float*)p)[i];
}
template <int MODE> __device__ __forceinline__ void st(void* p, int64_t i, float v)
{
    if (MODE) ((uint16_t*)p)[i] = (uint16_t)(__float_as_uint(v) >> 16);   // v is already a bf16 value
    else ((float*)p)[i] = v;
}

template <int MODE>
__global__ __launch_bounds__(256) void scalars_kernel(const void* __restrict__ x, void* __restrict__ s, int64_t nblocks)
{
    for (int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x; b < nblocks; b += (int64_t)gridDim.x * 256) {
        float m = 0.0f;
#pragma unroll
        for (int j = 0; j < kBlock; ++j) m = fmaxf(m, fabsf(ld<MODE>(x, b * kBlock + j)));
        st<MODE>(s, b, rd<MODE>(rd<MODE>(m / 6.0f) + 1e-9f));
    }
}

template <int MODE, bool SR>
__global__ __launch_bounds__(256) void values_kernel(const void* __restrict__ x, const void* __restrict__ s,
                                                     const void* __restrict__ noise, uint64_t seed, uint64_t offset,
                                                     void* __restrict__ out, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
        const float xv = ld<MODE>(x, i);
        const float h = rd<MODE>(ld<MODE>(s, i / kBlock) / 2.0f);
        float u = 0.0f;
        if (SR) {
            if (noise) u = ld<MODE>(noise, i);
            else {
                const uint4 r = Philox::draw(offset + (uint64_t)(i >> 2), seed);
                const uint32_t w = (i & 3) == 0 ? r.x : (i & 3) == 1 ? r.y : (i & 3) == 2 ? r.z : r.w;
                u = uniform_from_bits<MODE>(w);
            }
        }
        const float r = code_literal<MODE, SR>(fabsf(xv), h, u);
        // expand (quant.py:127), then * sign / 2
        const float v = r + (fmaxf(r - 4.0f, 0.0f) + fmaxf(r - 6.0f, 0.0f) * 2.0f);
        const float sg = xv > 0.0f ? 1.0f : (xv < 0.0f ? -1.0f : 0.0f);
        st<MODE>(out, i, (v * sg) / 2.0f);
    }
}

// max |s| over the tensor, single workgroup (scalar tensors are small: 1/16 of the data)
template <int MODE>
__global__ __launch_bounds__(1024) void smax_kernel(const void* __restrict__ s, int64_t nblocks, float* __restrict__ smax)
{
    __shared__ float part[16];
    float m = 0.0f;
    for (int64_t b = threadIdx.x; b < nblocks; b += 1024) m = fmaxf(m, fabsf(ld<MODE>(s, b)));
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; ++w) m = fmaxf(m, part[w]);
        *smax = m;
    }
}

template <int MODE>
__global__ __launch_bounds__(256) void rquant_kernel(const void* __restrict__ xq, void* __restrict__ s,
                                                     const float* __restrict__ smax, void* __restrict__ out, int64_t nblocks)
{
    const float unit = rd<MODE>(*smax / 448.0f);                         // smax / 448
    for (int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x; b < nblocks; b += (int64_t)gridDim.x * 256) {
        const float t = rd<MODE>(ld<MODE>(s, b) / unit);                  // s /= smax / 448   (in place)
        st<MODE>(s, b, t);
        const float dq = rd<MODE>(e4m3_value(e4m3_byte(t)) * unit);       // e4m3 round trip, *= smax / 448
#pragma unroll
        for (int j = 0; j < kBlock; ++j) st<MODE>(out, b * kBlock + j, rd<MODE>(ld<MODE>(xq, b * kBlock + j) * dq));
    }
}

static int grid1(int64_t items)
{
    int64_t g = (items + 255) / 256;
    const int64_t cap = (int64_t)device_cus() * 16;
    return (int)(g < 1 ? 1 : (g > cap ? cap : g));
}

int block_scalars(const void* x, int64_t rows, int64_t cols, int mode, void* s, hipStream_t st_)
{
    if (rows < 0 || cols < 0 || (mode != 0 && mode != 1)) return METIS_E_ARG;
    if (cols % kBlock) return METIS_E_SHAPE;
    const int64_t nb = rows * cols / kBlock;
    if (nb == 0) return METIS_OK;
    if (!x || !s) return METIS_E_ARG;
    if (mode == 0) hipLaunchKernelGGL(scalars_kernel<0>, dim3(grid1(nb)), dim3(256), 0, st_, x, s, nb);
    else hipLaunchKernelGGL(scalars_kernel<1>, dim3(grid1(nb)), dim3(256), 0, st_, x, s, nb);
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

int quant_values(const void* x, const void* s, int64_t rows, int64_t cols, int mode, int sr, const void* noise,
                 uint64_t seed, uint64_t offset, void* out, hipStream_t st_)
{
    if (rows < 0 || cols < 0 || (mode != 0 && mode != 1)) return METIS_E_ARG;
    if (cols % kBlock) return METIS_E_SHAPE;
    const int64_t n = rows * cols;
    if (n == 0) return METIS_OK;
    if (!x || !s || !out) return METIS_E_ARG;
    const int g = grid1(n);
#define METIS_V(M, S) hipLaunchKernelGGL((values_kernel<M, S>), dim3(g), dim3(256), 0, st_, x, s, noise, seed, offset, out, n)
    if (mode == 0) { if (sr) METIS_V(0, true); else METIS_V(0, false); }
    else { if (sr) METIS_V(1, true); else METIS_V(1, false); }
#undef METIS_V
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

int rquant_values(const void* xq, void* s, int64_t rows, int64_t cols, int mode, void* out, float* scratch,
                  hipStream_t st_)
{
    if (rows < 0 || cols < 0 || (mode != 0 && mode != 1)) return METIS_E_ARG;
    if (cols % kBlock) return METIS_E_SHAPE;
    const int64_t nb = rows * cols / kBlock;
    if (nb == 0) return METIS_OK;
    if (!xq || !s || !out || !scratch) return METIS_E_ARG;
    if (mode == 0) {
        hipLaunchKernelGGL(smax_kernel<0>, dim3(1), dim3(1024), 0, st_, (const void*)s, nb, scratch);
        hipLaunchKernelGGL(rquant_kernel<0>, dim3(grid1(nb)), dim3(256), 0, st_, xq, s, scratch, out, nb);
    } else {
        hipLaunchKernelGGL(smax_kernel<1>, dim3(1), dim3(1024), 0, st_, (const void*)s, nb, scratch);
        hipLaunchKernelGGL(rquant_kernel<1>, dim3(grid1(nb)), dim3(256), 0, st_, xq, s, scratch, out, nb);
    }
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

}  // namespace metis
