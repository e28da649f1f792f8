// NVFP4 quantizer kernels for gfx950: block-16 absmax -> E2M1 codes + E4M3 block scales + a
// binary32 tensor scale, round-to-nearest or stochastic rounding, row- or column-blocked.
//
// Replaces the eager op chain of src/Metis/Metis/quant.py:6-36 (RNE) and 273-308 + 137-147
// (stochastic rounding).  HBM-bound integer/byte work: one coalesced read of the bf16 input,
// 0.5 B/element of codes and 1/16 B/element of scales written.
//
// Two-phase structure forced by the arithmetic: the codes depend only on the block's own raw
// scalar (quant.py:27), the scale bytes on the tensor-wide maximum (quant.py:21-23).  Phase 1
// writes codes, parks each block's maximum as bf16 (2 B per block) and publishes one partial
// maximum per workgroup; phase 2 turns the parked maxima into E4M3 bytes.
#include "metis_device.h"
#include "metis_host.h"
#include "nvfp4_encode.h"

namespace metis {

// ---------------------------------------------------------------------------------------------
// Phase 1: codes + parked block maxima + per-workgroup maximum.  One block of 16 per thread per
// iteration.  Row layout: thread i <-> block i (32 contiguous bytes, two 16-byte loads).
// Column layout: thread i <-> (block-row b = i / cols, column c = i % cols) so that a wave reads
// 64 consecutive columns of each of the 16 rows.
// ---------------------------------------------------------------------------------------------
template <int MODE, bool SR, bool COL>
__global__ __launch_bounds__(256) void quant_codes_kernel(
    const uint16_t* __restrict__ x, uint32_t rows, uint32_t cols, int64_t ld, const void* __restrict__ noise,
    uint64_t seed, uint64_t offset, uint2* __restrict__ codes, uint16_t* __restrict__ ws_amax,
    uint32_t* __restrict__ ws_gmax, uint32_t nblocks)
{
    float gmax = 0.0f;
    const uint32_t nbpr = cols / kBlock;      // row layout: blocks per row
    const uint32_t nbc = rows / kBlock;       // column layout: blocks per column
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < nblocks; i += gridDim.x * 256u) {
        float v[kBlock], u[kBlock] = {};
        uint32_t ob;
        if constexpr (!COL) {
            ob = i;
            const uint32_t row = i / nbpr, cb = i - row * nbpr;
            const uint4* p = reinterpret_cast<const uint4*>(x + (int64_t)row * ld + (int64_t)cb * kBlock);
            unpack16(p[0], p[1], v);
            if (SR && noise) {
#pragma unroll
                for (int j = 0; j < kBlock; ++j) {
                    int64_t e = (int64_t)i * kBlock + j;
                    u[j] = MODE ? bf16_lo(((const uint16_t*)noise)[e]) : ((const float*)noise)[e];
                }
            }
        } else {
            const uint32_t b = i / cols, c = i - b * cols;
            ob = c * nbc + b;
#pragma unroll
            for (int j = 0; j < kBlock; ++j) v[j] = bf16_lo(x[(int64_t)(b * kBlock + j) * ld + c]);
            if (SR && noise) {
#pragma unroll
                for (int j = 0; j < kBlock; ++j) {
                    int64_t e = (int64_t)(b * kBlock + j) * cols + c;
                    u[j] = MODE ? bf16_lo(((const uint16_t*)noise)[e]) : ((const float*)noise)[e];
                }
            }
        }
        if (SR && !noise) philox16<MODE>(seed, offset, ob, u);
        const float am = block_amax(v);
        gmax = fmaxf(gmax, am);
        ws_amax[ob] = (uint16_t)(__float_as_uint(am) >> 16);          // am is a bf16 value
        codes[ob] = encode_block<MODE, SR>(v, block_scalar<MODE>(am), u);
    }
    publish_group_max(gmax, ws_gmax);
}

// ---------------------------------------------------------------------------------------------
// Phase 2: tensor unit and E4M3 scale bytes (quant.py:21-23), four blocks per thread.
// Every workgroup folds the published partial maxima itself (a few KB from L2).
// ---------------------------------------------------------------------------------------------
template <int MODE>
__global__ __launch_bounds__(256) void quant_scales_kernel(const uint16_t* __restrict__ ws_amax,
                                                           const uint32_t* __restrict__ ws_gmax, uint32_t ngroups,
                                                           uint8_t* __restrict__ scales, float* __restrict__ unit_out,
                                                           uint32_t nblocks)
{
    __shared__ float smax[4];
    float m = 0.0f;
    for (uint32_t g = threadIdx.x; g < ngroups; g += 256u) m = fmaxf(m, __uint_as_float(ws_gmax[g]));
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) smax[threadIdx.x >> 6] = m;
    __syncthreads();
    const float amax = fmaxf(fmaxf(smax[0], smax[1]), fmaxf(smax[2], smax[3]));
    // max over blocks of scalar(amax_block) = scalar(max amax_block): the scalar map is monotone
    const float unit = rd<MODE>(block_scalar<MODE>(amax) / 448.0f);
    if (blockIdx.x == 0 && threadIdx.x == 0) *unit_out = unit;

    const uint32_t nquads = (nblocks + 3u) / 4u;
    for (uint32_t q = blockIdx.x * 256u + threadIdx.x; q < nquads; q += gridDim.x * 256u) {
        const uint32_t base = q * 4u;
        if (base + 4u <= nblocks) {
            const uint2 a = *reinterpret_cast<const uint2*>(ws_amax + base);
            const float t0 = rd<MODE>(block_scalar<MODE>(bf16_lo(a.x)) / unit);
            const float t1 = rd<MODE>(block_scalar<MODE>(bf16_hi(a.x)) / unit);
            const float t2 = rd<MODE>(block_scalar<MODE>(bf16_lo(a.y)) / unit);
            const float t3 = rd<MODE>(block_scalar<MODE>(bf16_hi(a.y)) / unit);
            int w = __builtin_amdgcn_cvt_pk_fp8_f32(t0, t1, 0, false);
            w = __builtin_amdgcn_cvt_pk_fp8_f32(t2, t3, w, true);
            *reinterpret_cast<uint32_t*>(scales + base) = (uint32_t)w;
        } else {
            for (uint32_t k = base; k < nblocks; ++k) {
                const float s = block_scalar<MODE>(__uint_as_float((uint32_t)ws_amax[k] << 16));
                scales[k] = (uint8_t)e4m3_byte(rd<MODE>(s / unit));
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Dequantize: ((v * sign) / 2) * (e4m3 * unit), quant.py:23-24 and 32-35.  Eight elements per thread.
// ---------------------------------------------------------------------------------------------
template <int MODE, int OUT_F32>
__global__ __launch_bounds__(256) void dequant_kernel(const uint32_t* __restrict__ codes, const uint8_t* __restrict__ scales,
                                                      const float* __restrict__ unit_p, void* __restrict__ out, int64_t noct)
{
    const float unit = *unit_p;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < noct; i += (int64_t)gridDim.x * 256) {
        const uint32_t c = codes[i];
        const float dq = rd<MODE>(e4m3_value(scales[i >> 1]) * unit);
        float o[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t nib = (c >> (4 * j)) & 0xfu, r = nib & 7u;
            // expand (quant.py:32-34): r + relu(r-4) + 2 relu(r-6)
            float v = (float)(r + (r > 4u ? r - 4u : 0u) + (r > 6u ? 2u * (r - 6u) : 0u));
            v = (nib & 8u) ? -v : v;
            o[j] = rd<MODE>((v * 0.5f) * dq);
        }
        if (OUT_F32) {
            float4* p = reinterpret_cast<float4*>(out) + i * 2;
            p[0] = make_float4(o[0], o[1], o[2], o[3]);
            p[1] = make_float4(o[4], o[5], o[6], o[7]);
        } else {
            uint4 w;
            w.x = bf16_bits(o[0]) | (bf16_bits(o[1]) << 16);
            w.y = bf16_bits(o[2]) | (bf16_bits(o[3]) << 16);
            w.z = bf16_bits(o[4]) | (bf16_bits(o[5]) << 16);
            w.w = bf16_bits(o[6]) | (bf16_bits(o[7]) << 16);
            reinterpret_cast<uint4*>(out)[i] = w;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------
static int grid_for(uint32_t work_items)
{
    int64_t g = ((int64_t)work_items + 255) / 256;
    const int64_t cap = (int64_t)device_cus() * 8;           // 8 workgroups of 256 per CU are resident
    if (g > cap) g = cap;
    if (g > kMaxGroups) g = kMaxGroups;
    return g < 1 ? 1 : (int)g;
}

int launch_scales(int mode, const Workspace& ws, uint32_t ngroups, void* scales, float* unit, uint32_t nblocks,
                  hipStream_t st)
{
    const int g2 = grid_for((nblocks + 3) / 4);
    if (mode == 0)
        hipLaunchKernelGGL((quant_scales_kernel<0>), dim3(g2), dim3(256), 0, st, ws.amax, ws.gmax, ngroups,
                           (uint8_t*)scales, unit, nblocks);
    else
        hipLaunchKernelGGL((quant_scales_kernel<1>), dim3(g2), dim3(256), 0, st, ws.amax, ws.gmax, ngroups,
                           (uint8_t*)scales, unit, nblocks);
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

template <int MODE, bool SR, bool COL>
static int launch_quant(const void* x, int64_t rows, int64_t cols, int64_t ld, const void* noise, uint64_t seed,
                        uint64_t offset, void* codes, void* scales, float* unit, const Workspace& ws, hipStream_t st)
{
    const uint32_t nblocks = (uint32_t)(rows * cols / kBlock);
    const int g1 = grid_for(nblocks);
    hipLaunchKernelGGL((quant_codes_kernel<MODE, SR, COL>), dim3(g1), dim3(256), 0, st, (const uint16_t*)x,
                       (uint32_t)rows, (uint32_t)cols, ld, noise, seed, offset, (uint2*)codes, ws.amax, ws.gmax, nblocks);
    return launch_scales(MODE, ws, (uint32_t)g1, scales, unit, nblocks, st);
}

int quantize(const void* x, int64_t rows, int64_t cols, int64_t ld, int mode, bool sr, bool col, const void* noise,
             uint64_t seed, uint64_t offset, void* codes, void* scales, float* unit, void* workspace,
             size_t workspace_bytes, hipStream_t st)
{
    if (rows < 0 || cols < 0 || ld < cols) return METIS_E_ARG;
    if (mode != METIS_MODE_P32 && mode != METIS_MODE_PB16) return METIS_E_ARG;
    if ((col ? rows : cols) % kBlock) return METIS_E_SHAPE;
    if (rows == 0 || cols == 0) return METIS_OK;              // nothing to read or write, unit untouched
    if (!x || !codes || !scales || !unit) return METIS_E_ARG;
    if (rows * cols / kBlock >= (int64_t)1 << 31) return METIS_E_ARG;
    if (!col && ((ld % 8) || ((uintptr_t)x % 16))) return METIS_E_ARG;     // 16-byte vector loads
    if (((uintptr_t)codes % 8) || ((uintptr_t)scales % 4)) return METIS_E_ARG;
    Workspace ws;
    int rc = carve_workspace(workspace, workspace_bytes, rows, cols, &ws);
    if (rc != METIS_OK) return rc;
#define METIS_Q(M, S, C) return launch_quant<M, S, C>(x, rows, cols, ld, noise, seed, offset, codes, scales, unit, ws, st)
    if (mode == 0) {
        if (!sr) { if (!col) METIS_Q(0, false, false); else METIS_Q(0, false, true); }
        else { if (!col) METIS_Q(0, true, false); else METIS_Q(0, true, true); }
    } else {
        if (!sr) { if (!col) METIS_Q(1, false, false); else METIS_Q(1, false, true); }
        else { if (!col) METIS_Q(1, true, false); else METIS_Q(1, true, true); }
    }
#undef METIS_Q
}

int dequantize(const void* codes, const void* scales, const float* unit, int64_t rows, int64_t cols, int mode, void* out,
               int out_dtype, hipStream_t st)
{
    if (rows < 0 || cols < 0) return METIS_E_ARG;
    if (mode != METIS_MODE_P32 && mode != METIS_MODE_PB16) return METIS_E_ARG;
    if (out_dtype != METIS_DTYPE_BF16 && out_dtype != METIS_DTYPE_F32) return METIS_E_ARG;
    if (cols % kBlock) return METIS_E_SHAPE;
    if (rows == 0 || cols == 0) return METIS_OK;
    if (!codes || !scales || !unit || !out) return METIS_E_ARG;
    if (((uintptr_t)codes % 4) || ((uintptr_t)out % 16)) return METIS_E_ARG;
    const int64_t noct = rows * cols / 8;
    if (noct == 0) return METIS_OK;
    int64_t g = (noct + 255) / 256;
    const int64_t cap = (int64_t)device_cus() * 16;
    if (g > cap) g = cap;
#define METIS_D(M, F) hipLaunchKernelGGL((dequant_kernel<M, F>), dim3((int)g), dim3(256), 0, st, (const uint32_t*)codes, \
                                         (const uint8_t*)scales, unit, out, noct)
    if (mode == 0) { if (out_dtype == METIS_DTYPE_F32) METIS_D(0, 1); else METIS_D(0, 0); }
    else { if (out_dtype == METIS_DTYPE_F32) METIS_D(1, 1); else METIS_D(1, 0); }
#undef METIS_D
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

}  // namespace metis
