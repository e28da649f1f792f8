// Fused RMSNorm -> NVFP4 quantization for gfx950: one HBM read of the hidden states.
//
// RMSNorm: src/Metis/models/llama.py:23-31 with a bf16 weight (binary32 x * rsqrt(mean(x^2)+eps),
// rounded to bf16, times gamma, rounded to bf16).  The quantizer then runs on those bf16 values
// exactly as nvfp4_quant.hip does (src/Metis/Metis/quant.py:6-36); the reference reaches it via
// LinearLowbitFunction.quantize_input (src/Metis/Metis/bitlinear.py:371-393).
//
// One workgroup of 256 threads owns a row at a time; thread t holds blocks t, t+256, ... of the
// row in registers, so the row is read once.  The sum of squares is reduced across lanes with
// DPP shuffles and across the four waves through LDS.
#include "metis_device.h"
#include "metis_host.h"
#include "nvfp4_encode.h"

namespace metis {

template <int MODE, int NBT, bool WRITE_NORMED>
__global__ __launch_bounds__(256) void rmsnorm_quant_kernel(const uint16_t* __restrict__ x,
                                                            const uint16_t* __restrict__ gamma, float eps,
                                                            uint32_t rows, uint32_t cols, uint16_t* __restrict__ normed,
                                                            uint2* __restrict__ codes, uint16_t* __restrict__ ws_amax,
                                                            uint32_t* __restrict__ ws_gmax, uint32_t fill_to)
{
    __shared__ float part[2][4];
    const uint32_t nbpr = cols / kBlock;
    const float inv_is_div = (float)cols;                     // mean = sum / cols (a division, as torch.mean)
    float gmax = 0.0f;
    uint32_t parity = 0;
    // gamma of the thread's first block stays in registers for every row (all of it when cols <= 4096)
    float g0[kBlock] = {};
    if (threadIdx.x < nbpr) {
        const uint4* g = reinterpret_cast<const uint4*>(gamma + (int64_t)threadIdx.x * kBlock);
        unpack16(g[0], g[1], g0);
    }
    // the next row's bytes are requested before the current row is reduced and encoded
    uint4 raw[NBT][2];
    auto request = [&](uint32_t row) {
#pragma unroll
        for (int k = 0; k < NBT; ++k) {
            const uint32_t cb = threadIdx.x + k * 256u;
            if (cb < nbpr) {
                const uint4* p = reinterpret_cast<const uint4*>(x + (int64_t)row * cols + (int64_t)cb * kBlock);
                raw[k][0] = p[0];
                raw[k][1] = p[1];
            }
        }
    };
    if (blockIdx.x < rows) request(blockIdx.x);
    for (uint32_t row = blockIdx.x; row < rows; row += gridDim.x, parity ^= 1u) {
        float v[NBT][kBlock];
        float ss = 0.0f;
#pragma unroll
        for (int k = 0; k < NBT; ++k) {
            const uint32_t cb = threadIdx.x + k * 256u;
            if (cb < nbpr) {
                unpack16(raw[k][0], raw[k][1], v[k]);
#pragma unroll
                for (int j = 0; j < kBlock; ++j) ss = fmaf(v[k][j], v[k][j], ss);
            }
        }
        if (row + gridDim.x < rows) request(row + gridDim.x);
        ss = wave_sum(ss);
        if ((threadIdx.x & 63) == 0) part[parity][threadIdx.x >> 6] = ss;
        __syncthreads();                                      // the other parity is free again after this barrier
        const float total = (part[parity][0] + part[parity][1]) + (part[parity][2] + part[parity][3]);
        const float rstd = 1.0f / sqrtf(total / inv_is_div + eps);
#pragma unroll
        for (int k = 0; k < NBT; ++k) {
            const uint32_t cb = threadIdx.x + k * 256u;
            if (cb < nbpr) {
                float gm[kBlock], n[kBlock];
                if (k == 0) {
#pragma unroll
                    for (int j = 0; j < kBlock; ++j) gm[j] = g0[j];
                } else {
                    const uint4* g = reinterpret_cast<const uint4*>(gamma + (int64_t)cb * kBlock);
                    unpack16(g[0], g[1], gm);
                }
                // bf16(bf16(x * rstd) * gamma), two elements per conversion; the packed pairs are the normed output
                uint32_t w[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t h = rb_pair(v[k][2 * j] * rstd, v[k][2 * j + 1] * rstd);
                    w[j] = rb_pair(bf16_lo(h) * gm[2 * j], bf16_hi(h) * gm[2 * j + 1]);
                    n[2 * j] = bf16_lo(w[j]);
                    n[2 * j + 1] = bf16_hi(w[j]);
                }
                const uint32_t ob = row * nbpr + cb;
                if (WRITE_NORMED) {
                    uint4* o = reinterpret_cast<uint4*>(normed + (int64_t)ob * kBlock);
                    o[0] = make_uint4(w[0], w[1], w[2], w[3]);
                    o[1] = make_uint4(w[4], w[5], w[6], w[7]);
                }
                const float am = block_amax(n);
                gmax = fmaxf(gmax, am);
                ws_amax[ob] = (uint16_t)(__float_as_uint(am) >> 16);
                const float none[kBlock] = {};
                codes[ob] = encode_block<MODE, false>(n, block_scalar<MODE>(am), none);
            }
        }
    }
    publish_group_max(gmax, ws_gmax, fill_to);
}

// deferred: stop after the main kernel; `workspace` is then the caller-owned parked data of the deferred form
// (nvfp4_quant.hip) and scales / unit are not written.
int rmsnorm_quantize(const void* x, const void* gamma, float eps, int64_t rows, int64_t cols, int mode, void* normed,
                     void* codes, void* scales, float* unit, void* workspace, size_t workspace_bytes, hipStream_t st, bool deferred)
{
    if (rows < 0 || cols < 0) return METIS_E_ARG;
    if (mode != METIS_MODE_P32 && mode != METIS_MODE_PB16) return METIS_E_ARG;
    if (cols % kBlock) return METIS_E_SHAPE;
    if (rows == 0 || cols == 0) return METIS_OK;
    if (!x || !gamma || !codes || (!deferred && (!scales || !unit))) return METIS_E_ARG;
    if (cols > 256 * kBlock * 4) return METIS_E_ARG;          // a row is held in registers: at most 16384 columns
    if (rows * cols / kBlock >= (int64_t)1 << 31) return METIS_E_ARG;
    if (((uintptr_t)x % 16) || ((uintptr_t)gamma % 16) || ((uintptr_t)codes % 8) || ((uintptr_t)scales % 8) ||
        (normed && ((uintptr_t)normed % 16)))
        return METIS_E_ARG;
    Workspace ws;
    int rc = deferred ? carve_deferred(workspace, workspace_bytes, rows, cols, &ws) : carve_workspace(workspace, workspace_bytes, rows, cols, &ws);
    if (rc != METIS_OK) return rc;
    int64_t g = rows;
    const int64_t cap = (int64_t)device_cus() * 8;
    if (g > cap) g = cap;
    if (g > kMaxGroups) g = kMaxGroups;
    if (deferred && g > (int64_t)kDeferredPartials) g = kDeferredPartials;
    const uint32_t fill_to = deferred ? kDeferredPartials : 0u;
    const int nbt = (int)((cols / kBlock + 255) / 256);
#define METIS_R(M, NBT, W) hipLaunchKernelGGL((rmsnorm_quant_kernel<M, NBT, W>), dim3((int)g), dim3(256), 0, st, \
        (const uint16_t*)x, (const uint16_t*)gamma, eps, (uint32_t)rows, (uint32_t)cols, (uint16_t*)normed, (uint2*)codes, \
        ws.amax, ws.gmax, fill_to)
#define METIS_RN(M, W) do { if (nbt <= 1) METIS_R(M, 1, W); else if (nbt == 2) METIS_R(M, 2, W); else METIS_R(M, 4, W); } while (0)
    if (mode == 0) { if (normed) METIS_RN(0, true); else METIS_RN(0, false); }
    else { if (normed) METIS_RN(1, true); else METIS_RN(1, false); }
#undef METIS_RN
#undef METIS_R
    if (hipGetLastError() != hipSuccess) return METIS_E_LAUNCH;
    if (deferred) return METIS_OK;
    return launch_scales(mode, ws, (uint32_t)g, scales, unit, (uint32_t)(rows * cols / kBlock), st);
}

}  // namespace metis
