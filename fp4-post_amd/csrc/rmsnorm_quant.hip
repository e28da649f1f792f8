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

// ---------------------------------------------------------------------------------------------
// Rows of at most 4096 columns: one WAVE per row, no barrier and no LDS traffic for the reduction.  Lane l holds the
// 16-byte chunks l, l + 64, ... of the row (8 elements: half a scale block; lanes 2m and 2m + 1 share a block), so
// every load and store instruction of the wave covers consecutive bytes: a KiB of the row in, a KiB of the normed
// row out, 256 bytes of codes.  (Thread-per-block stores of the normed row, 16 bytes at a 32-byte lane stride, held
// this kernel's byte mix to 5.2 TB/s; whole lines written with the non-temporal hint reach 7.)  The sum of squares is
// taken on the packed pairs (v_dot2_f32_bf16) and folded across the wave with DPP moves; the product with gamma is a
// v_dot2_f32_bf16 of the packed bf16(x * rstd) pair against gamma with the other half masked off -- the exact product
// of the two bf16 values, no unpacking (subnormal products are rounded differently by that instruction and a zero
// product comes out as +0.0: both below anything the normed tensor's consumers can tell apart).  gamma is staged in
// LDS once per workgroup in that masked form; the block maximum is one DPP exchange between the two lanes of a block.
// ---------------------------------------------------------------------------------------------
typedef __bf16 metis_bf16pair_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float c)
{
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(metis_bf16pair_t, a), __builtin_bit_cast(metis_bf16pair_t, b), c, false);
}
template <int CTRL> __device__ __forceinline__ float dpp_f32(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
// sum over the 64 lanes, the same value in every lane
__device__ __forceinline__ float wave_sum_dpp(float v)
{
    v += dpp_f32<0xB1>(v);           // quad_perm [1,0,3,2]
    v += dpp_f32<0x4E>(v);           // quad_perm [2,3,0,1]
    v += dpp_f32<0x141>(v);          // row_half_mirror
    v += dpp_f32<0x140>(v);          // row_mirror: every lane of a row of 16 holds the row's sum
    const int b = __builtin_bit_cast(int, v);                 // (the builtin takes an integer: pass the bits, not the value)
    const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)), r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
    const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)), r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
    return (r0 + r1) + (r2 + r3);
}
typedef uint32_t metis_u32x4_t __attribute__((ext_vector_type(4)));

template <int MODE, int NL, bool WRITE_NORMED>
__global__ __launch_bounds__(256) void rmsnorm_quant_rows_kernel(const uint4* __restrict__ x, const uint4* __restrict__ gamma, float eps,
                                                                 uint32_t rows, uint32_t cols, metis_u32x4_t* __restrict__ normed,
                                                                 uint32_t* __restrict__ codes, uint16_t* __restrict__ ws_amax,
                                                                 uint32_t* __restrict__ ws_gmax, uint32_t fill_to)
{
    __shared__ uint4 g_a[NL * 64], g_b[NL * 64];              // gamma pairs 0, 1 and 2, 3 of every chunk, each as {low only, high only}
    __shared__ uint32_t table[MODE == 0 ? kQuotientTableWords : 4];
    const uint32_t cpr = cols / 8u;                           // 16-byte chunks per row (even: cols % 16 == 0)
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const float fcols = (float)cols;
    const uint32_t wstep = gridDim.x * 4u;
    uint32_t row = blockIdx.x * 4u + wave;
    uint4 raw[NL];
    auto request = [&](uint32_t r) {
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            const uint32_t c = i * 64u + lane;
            if (c < cpr) raw[i] = x[(size_t)r * cpr + c];
        }
    };
#pragma unroll
    for (int i = 0; i < NL; ++i) raw[i] = make_uint4(0u, 0u, 0u, 0u);
    if (row < rows) request(row);
    for (uint32_t c = threadIdx.x; c < cpr; c += 256u) {
        const uint4 g = gamma[c];
        g_a[c] = make_uint4(g.x & 0xffffu, g.x & 0xffff0000u, g.y & 0xffffu, g.y & 0xffff0000u);
        g_b[c] = make_uint4(g.z & 0xffffu, g.z & 0xffff0000u, g.w & 0xffffu, g.w & 0xffff0000u);
    }
    if constexpr (MODE == 0) stage_quotient_table(table);
    else __syncthreads();
    float gmax = 0.0f;
    for (; row < rows; row += wstep) {
        uint4 cur[NL];
        float ss = 0.0f;
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            cur[i] = raw[i];
            ss = dot2_bf16(cur[i].x, cur[i].x, ss);
            ss = dot2_bf16(cur[i].y, cur[i].y, ss);
            ss = dot2_bf16(cur[i].z, cur[i].z, ss);
            ss = dot2_bf16(cur[i].w, cur[i].w, ss);
        }
        if (row + wstep < rows) request(row + wstep);           // the next row is in flight while this one is encoded
        const float total = wave_sum_dpp(ss);
        const float rstd = 1.0f / sqrtf(total / fcols + eps);
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            const uint32_t c = i * 64u + lane;
            if (i * 64u >= cpr) break;                         // wave-uniform: chunks beyond the row
            if (c < cpr) {
                const uint32_t in[4] = {cur[i].x, cur[i].y, cur[i].z, cur[i].w};
                const uint4 ga = g_a[c], gb = g_b[c];
                const uint32_t gl[4] = {ga.x, ga.z, gb.x, gb.z}, gh[4] = {ga.y, ga.w, gb.y, gb.w};
                uint32_t w[4];
                float n[8];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    // bf16(bf16(x * rstd) * gamma), two elements per conversion; the packed pairs are the normed output
                    const uint32_t h = rb_pair(bf16_lo(in[j]) * rstd, bf16_hi(in[j]) * rstd);
                    w[j] = rb_pair(dot2_bf16(h, gl[j], 0.0f), dot2_bf16(h, gh[j], 0.0f));
                    n[2 * j] = bf16_lo(w[j]);
                    n[2 * j + 1] = bf16_hi(w[j]);
                }
                const size_t at = (size_t)row * cpr + c;
                if (WRITE_NORMED) __builtin_nontemporal_store((metis_u32x4_t){w[0], w[1], w[2], w[3]}, normed + at);
                float hm = amax3(0.0f, n[0], n[1]);
                hm = amax3(hm, n[2], n[3]);
                hm = amax3(hm, n[4], n[5]);
                hm = amax3(hm, n[6], n[7]);
                const float am = fmaxf(hm, dpp_f32<0xB1>(hm));  // the other half of the block sits in the neighbouring lane
                gmax = fmaxf(gmax, am);
                if ((lane & 1u) == 0u) ws_amax[at >> 1] = (uint16_t)(__float_as_uint(am) >> 16);
                uint32_t cw[1];
                if constexpr (MODE == 0) encode_rne_p32_tbl<8>(n, am, block_scalar<0>(am), table, cw);
                else encode_rne_pb16_n<8>(n, block_scalar<1>(am), cw);
                codes[at] = cw[0];
            }
        }
    }
    publish_group_max(gmax, ws_gmax, fill_to);
}

// ---------------------------------------------------------------------------------------------
// RMSNorm with the column sums of its output, for the mean mode (the reference's default arguments,
// src/grpo/grpo.py:66-69): there the activation is quantized as mean + QDQ(x - mean) with the column mean over tokens
// (src/Metis/Metis/bitlinear.py:311-336), so the quantizer needs the mean of the WHOLE normed tensor before it can
// start.  This kernel is the norm of rmsnorm_quant_rows_kernel (one wave per row, whole-line accesses) and leaves, per
// workgroup, the sums of the normed bf16 values of its rows, column by column, in a fixed order: rows in order within
// a wave, then the four waves in order.  rmsnorm_colmean_finish_kernel adds the workgroups' partial rows in order and
// applies the mean's division and rounding (and the running mean of decode calls) as column_mean_finish_kernel does.
// ---------------------------------------------------------------------------------------------
template <int NL>
__global__ __launch_bounds__(256) void rmsnorm_colsum_rows_kernel(const uint4* __restrict__ x, const uint4* __restrict__ gamma, float eps,
                                                                  uint32_t rows, uint32_t cols, metis_u32x4_t* __restrict__ normed,
                                                                  float* __restrict__ partial)
{
    __shared__ uint4 g_a[NL * 64], g_b[NL * 64];
    __shared__ float4 sums[NL * 64][2];                        // column sums of the workgroup, chunk by chunk
    const uint32_t cpr = cols / 8u;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const float fcols = (float)cols;
    const uint32_t wstep = gridDim.x * 4u;
    uint32_t row = blockIdx.x * 4u + wave;
    uint4 raw[NL];
    auto request = [&](uint32_t r) {
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            const uint32_t c = i * 64u + lane;
            if (c < cpr) raw[i] = x[(size_t)r * cpr + c];
        }
    };
#pragma unroll
    for (int i = 0; i < NL; ++i) raw[i] = make_uint4(0u, 0u, 0u, 0u);
    if (row < rows) request(row);
    for (uint32_t c = threadIdx.x; c < cpr; c += 256u) {
        const uint4 g = gamma[c];
        g_a[c] = make_uint4(g.x & 0xffffu, g.x & 0xffff0000u, g.y & 0xffffu, g.y & 0xffff0000u);
        g_b[c] = make_uint4(g.z & 0xffffu, g.z & 0xffff0000u, g.w & 0xffffu, g.w & 0xffff0000u);
    }
    __syncthreads();
    float acc[NL][8];
#pragma unroll
    for (int i = 0; i < NL; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = 0.0f;
    for (; row < rows; row += wstep) {
        uint4 cur[NL];
        float ss = 0.0f;
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            cur[i] = raw[i];
            ss = dot2_bf16(cur[i].x, cur[i].x, ss);
            ss = dot2_bf16(cur[i].y, cur[i].y, ss);
            ss = dot2_bf16(cur[i].z, cur[i].z, ss);
            ss = dot2_bf16(cur[i].w, cur[i].w, ss);
        }
        if (row + wstep < rows) request(row + wstep);
        const float total = wave_sum_dpp(ss);
        const float rstd = 1.0f / sqrtf(total / fcols + eps);
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            const uint32_t c = i * 64u + lane;
            if (i * 64u >= cpr) break;
            if (c < cpr) {
                const uint32_t in[4] = {cur[i].x, cur[i].y, cur[i].z, cur[i].w};
                const uint4 ga = g_a[c], gb = g_b[c];
                const uint32_t gl[4] = {ga.x, ga.z, gb.x, gb.z}, gh[4] = {ga.y, ga.w, gb.y, gb.w};
                uint32_t w[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t h = rb_pair(bf16_lo(in[j]) * rstd, bf16_hi(in[j]) * rstd);
                    w[j] = rb_pair(dot2_bf16(h, gl[j], 0.0f), dot2_bf16(h, gh[j], 0.0f));
                    acc[i][2 * j] += bf16_lo(w[j]);
                    acc[i][2 * j + 1] += bf16_hi(w[j]);
                }
                __builtin_nontemporal_store((metis_u32x4_t){w[0], w[1], w[2], w[3]}, normed + (size_t)row * cpr + c);
            }
        }
    }
    // the four waves' sums, added in wave order
#pragma unroll 1
    for (uint32_t v = 0; v < 4u; ++v) {
        if (wave == v) {
#pragma unroll
            for (int i = 0; i < NL; ++i) {
                const uint32_t c = i * 64u + lane;
                if (c < cpr) {
                    float4 lo = make_float4(acc[i][0], acc[i][1], acc[i][2], acc[i][3]), hi = make_float4(acc[i][4], acc[i][5], acc[i][6], acc[i][7]);
                    if (v) {
                        const float4 pl = sums[c][0], ph = sums[c][1];
                        lo = make_float4(pl.x + lo.x, pl.y + lo.y, pl.z + lo.z, pl.w + lo.w);
                        hi = make_float4(ph.x + hi.x, ph.y + hi.y, ph.z + hi.z, ph.w + hi.w);
                    }
                    sums[c][0] = lo;
                    sums[c][1] = hi;
                }
            }
        }
        __syncthreads();
    }
    float4* out = reinterpret_cast<float4*>(partial + (size_t)blockIdx.x * cols);
    for (uint32_t q = threadIdx.x; q < cpr * 2u; q += 256u) out[q] = sums[q >> 1][q & 1u];
}

constexpr int kColmeanBatch = 8;
template <bool OUT_BF16>
__global__ __launch_bounds__(256) void rmsnorm_colmean_finish_kernel(const float* __restrict__ partial, uint32_t slabs, uint32_t cols,
                                                                     float count, void* __restrict__ out, const void* __restrict__ cached,
                                                                     float cached_count, float rows_f, float* __restrict__ out32)
{
    __shared__ float part[4][64];
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t c = blockIdx.x * 64u + lane;
    float s = 0.0f;
    if (c < cols) {
        // wave w adds the partial rows w, w + 4, ... in order, kColmeanBatch loads in flight at a time
        for (uint32_t k0 = wave; k0 < slabs; k0 += 4u * kColmeanBatch) {
            float v[kColmeanBatch];
#pragma unroll
            for (int b = 0; b < kColmeanBatch; ++b) {
                const uint32_t k = k0 + 4u * b;
                v[b] = k < slabs ? partial[(size_t)k * cols + c] : 0.0f;
            }
#pragma unroll
            for (int b = 0; b < kColmeanBatch; ++b) s += v[b];
        }
    }
    part[wave][lane] = s;
    __syncthreads();
    if (wave != 0 || c >= cols) return;
    s = (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);
    auto rnd = [](float x) { return OUT_BF16 ? __uint_as_float(bf16_bits(x) << 16) : x; };
    float m = rnd(s / count);
    if (cached) {                                              // weighted running mean of decode calls, bitlinear.py:316-323
        const float cm = OUT_BF16 ? __uint_as_float((uint32_t)static_cast<const uint16_t*>(cached)[c] << 16)
                                  : static_cast<const float*>(cached)[c];
        const float a = rnd(cm * cached_count), b = rnd(m * rows_f);
        m = rnd(rnd(a + b) / (cached_count + rows_f));
    }
    if (OUT_BF16) static_cast<uint16_t*>(out)[c] = (uint16_t)bf16_bits(m);
    else static_cast<float*>(out)[c] = m;
    if (out32) out32[c] = m;
}

static int colmean_grid(int64_t rows)
{
    int64_t g = (rows + 3) / 4;
    const int64_t cap = (int64_t)device_cus() * 2;           // the column sums cost registers: two waves per SIMD
    if (g > cap) g = cap;
    return g < 1 ? 1 : (int)g;
}

size_t rmsnorm_colmean_workspace_bytes(int64_t rows, int64_t cols)
{
    if (rows <= 0 || cols <= 0) return 0;
    return (size_t)colmean_grid(rows) * (size_t)cols * sizeof(float);
}

int rmsnorm_colmean(const void* x, const void* gamma, float eps, int64_t rows, int64_t cols, void* normed, void* mean, int mean_bf16,
                    const void* cached, int64_t cached_count, float* mean32, void* workspace, size_t workspace_bytes, hipStream_t st)
{
    if (rows <= 0 || cols <= 0) return METIS_E_ARG;
    if (cols % kBlock) return METIS_E_SHAPE;
    if (cols > 4096) return METIS_E_ARG;                      // one wave per row
    if (!x || !gamma || !normed || !mean) return METIS_E_ARG;
    if (cached && (cached_count < 0 || cached_count > (1 << 24) || ((uintptr_t)cached % (mean_bf16 ? 2 : 4)))) return METIS_E_ARG;
    if (((uintptr_t)x % 16) || ((uintptr_t)gamma % 16) || ((uintptr_t)normed % 16) || ((uintptr_t)mean % 4) || ((uintptr_t)mean32 % 4)) return METIS_E_ARG;
    if (!workspace || ((uintptr_t)workspace % 16) || workspace_bytes < rmsnorm_colmean_workspace_bytes(rows, cols)) return METIS_E_WORKSPACE;
    const int g = colmean_grid(rows);
    const int nl = (int)((cols / 8 + 63) / 64);
    float* partial = static_cast<float*>(workspace);
#define METIS_RC(NL) hipLaunchKernelGGL((rmsnorm_colsum_rows_kernel<NL>), dim3(g), dim3(256), 0, st, (const uint4*)x, (const uint4*)gamma, eps, \
        (uint32_t)rows, (uint32_t)cols, (metis_u32x4_t*)normed, partial)
    if (nl <= 2) METIS_RC(2); else if (nl <= 4) METIS_RC(4); else METIS_RC(8);
#undef METIS_RC
    if (hipGetLastError() != hipSuccess) return METIS_E_LAUNCH;
    const dim3 g2((unsigned)((cols + 63) / 64));
    if (mean_bf16)
        hipLaunchKernelGGL(rmsnorm_colmean_finish_kernel<true>, g2, dim3(256), 0, st, partial, (uint32_t)g, (uint32_t)cols, (float)rows, mean, cached,
                           (float)cached_count, (float)rows, mean32);
    else
        hipLaunchKernelGGL(rmsnorm_colmean_finish_kernel<false>, g2, dim3(256), 0, st, partial, (uint32_t)g, (uint32_t)cols, (float)rows, mean, cached,
                           (float)cached_count, (float)rows, mean32);
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

// deferred: stop after the main kernel; `workspace` is then the caller-owned parked data of the deferred form
// (nvfp4_quant.hip) and scales / unit are not written.
int rmsnorm_quantize(const void* x, const void* gamma, float eps, int64_t rows, int64_t cols, int mode, void* normed,
                     void* codes, void* scales, float* unit, void* workspace, size_t workspace_bytes, hipStream_t st, bool deferred,
                     void* decode)
{
    if (decode && (deferred || rows >= 256 || cols % 256)) return METIS_E_ARG;
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
    // Decode-sized calls take the workgroup-per-row kernel whatever the row length: with a wave per row, 64 rows are 16
    // workgroups and a lane encodes four blocks one after the other (64 x 3584: 6.6-7.3 against 3.9-4.2 us; same bits).
    if (cols <= 4096 && (rows >= 256 || measure_env("METIS_N_WAVE_PER_ROW"))) {
        // one wave per row
        int64_t g = (rows + 3) / 4;
        const int64_t cap = (int64_t)device_cus() * measure_int("METIS_N_WGPC", 3);
        if (g > cap) g = cap;
        if (g > kMaxGroups) g = kMaxGroups;
        if (deferred && g > (int64_t)kDeferredPartials) g = kDeferredPartials;
        const uint32_t fill_to = deferred ? kDeferredPartials : 0u;
        const int nl = (int)((cols / 8 + 63) / 64);
#define METIS_RW(M, NL, W) hipLaunchKernelGGL((rmsnorm_quant_rows_kernel<M, NL, W>), dim3((int)g), dim3(256), 0, st, (const uint4*)x, \
        (const uint4*)gamma, eps, (uint32_t)rows, (uint32_t)cols, (metis_u32x4_t*)normed, (uint32_t*)codes, ws.amax, ws.gmax, fill_to)
#define METIS_RWN(M, W) do { if (nl <= 2) METIS_RW(M, 2, W); else if (nl <= 4) METIS_RW(M, 4, W); else METIS_RW(M, 8, W); } while (0)
        if (mode == 0) { if (normed) METIS_RWN(0, true); else METIS_RWN(0, false); }
        else { if (normed) METIS_RWN(1, true); else METIS_RWN(1, false); }
#undef METIS_RWN
#undef METIS_RW
        if (hipGetLastError() != hipSuccess) return METIS_E_LAUNCH;
        if (deferred) return METIS_OK;
        if (decode) return launch_scales_decode(mode, ws, (uint32_t)g, codes, scales, unit, rows, cols, decode, st);
        return launch_scales(mode, ws, (uint32_t)g, scales, unit, (uint32_t)(rows * cols / kBlock), st);
    }
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
    if (decode) return launch_scales_decode(mode, ws, (uint32_t)g, codes, scales, unit, rows, cols, decode, st);
    return launch_scales(mode, ws, (uint32_t)g, scales, unit, (uint32_t)(rows * cols / kBlock), st);
}

}  // namespace metis
