// Block-scaled NVFP4 GEMM on operands that were expanded once, exactly, to binary16 in a tiled layout:
// the main loop is MFMA and LDS reads only, operand tiles travel HBM/L2 -> LDS by direct loads through a
// ring of stages with partial waits, one workgroup barrier per stage.
//
//   out[M,N] = ua*ub*2^16 * sum_k A16[m,k] B16[n,k]  +  sum_j T[m,j] U[n,j]  +  bias[n]
//
// Same contraction as gemm_nvfp4_large_kernel (metis_gemm.hip), which expands the packed operands inside its
// K loop; it replaces the same reference code: torch.matmul(input_, quantized_weight.T) (+ bias) of
// LinearLowbitFunction.forward (src/Metis/Metis/bitlinear.py:435-438) and the sum of the two branches of
// BitLinear.forward (752-760).  A16 = e2m1(code) * e4m3(scale) * 2^-8 is exact in binary16 (at most five
// significant bits), so both kernels feed the MFMAs the same values.
//
// Tiled layout ("xt") of an expanded [R, K] operand, K % 32 == 0: tiles of 16 rows x 32 k (1 KiB), tile
// (rb, kb) at byte ((rb * K/32) + kb) * 1024, rows padded to a multiple of 16 with zeros.  Inside a tile the
// 16-byte chunk c (8 consecutive k) of row q sits in slot q * 4 + (c ^ swz(q)).  One direct-to-LDS load
// instruction of a wave (64 lanes x 16 B) copies one tile: the global side reads 1 KiB of consecutive bytes
// (eight whole cache lines), the LDS side is written linearly, and the swizzle that makes the MFMA fragment
// reads (ds_read_b128, lane -> row) free of bank conflicts is already in the data.
#include "gemm_common.h"
#include "nvfp4_encode.h"
#include <stdlib.h>

namespace metis {

// swz(q) for row q of a tile (bits b1, b2, b3 of the row number): slot bit 0 = b2, slot bit 1 = b1 ^ b3.
// Any 8 consecutive rows then cover 8 different 16-byte units of a 128-byte bank period, and any 16
// consecutive rows 16 different units of a 256-byte period.
__host__ __device__ __forceinline__ int xt_swz(int q) { return ((q >> 2) & 1) | ((((q >> 1) ^ (q >> 3)) & 1) << 1); }

// ---------------------------------------------------------------------------------------------
// packed NVFP4 -> tiled 16-bit operands.  One wave per tile: lane l writes slot l (row l / 4).  A wave walks
// eight consecutive k tiles of one tile row, so the 128-byte lines of codes it touches are used whole.
// HBM-bound: 0.5625 B read, 2 B written per element.
//   PB16 = 0: binary16, e2m1(code) * e4m3(scale) * 2^-8, exact (the tensor unit is applied by the GEMM)
//   PB16 = 1: bf16, the reference's dequantized value with every op rounded to bf16
//             (src/Metis/Metis/quant.py:23-24, 32-35: bf16(bf16(e4m3 * unit) * v / 2)), unit included
// ---------------------------------------------------------------------------------------------
//   RHT: the packed tensor is a rotated one (NV recipe); every block of 16 is rotated back after dequantization,
//        (q H) / 16 * sign, as `_apply_hadamard_blocks(..., inverse=True)` does after the QDQ
//        (src/Metis/Metis/bitlinear.py:395-405, 577-585).  The two lanes that hold the halves of a block exchange
//        them and both run the 16-point butterflies.  PB16 = 0: the result is rounded to binary16 once (the sum of a
//        block needs at most 12 significant bits); PB16 = 1: dequantized values and result rounded to bf16 as the
//        reference's bf16 tensors are.
//   center (PB16 without RHT): the packed tensor is the centred residual of the mean mode; the operand is the
//        reference's me + QDQ(x - me) with the sum rounded to bf16 (src/Metis/Metis/bitlinear.py:330-333 in bf16
//        arithmetic): one bf16 value per column.
//   DEF: the quantizer stopped after its first phase (deferred scale bytes, nvfp4_quant.hip): `scales` holds one bf16
//        block maximum per block instead of E4M3 bytes, `partials` the partial tensor maxima.  The kernel forms the
//        tensor unit (written to unit_out by the first workgroup) and every scale byte itself, in the arithmetic the
//        tensor was quantized in (QMODE) -- the expressions of quant_scales_kernel, so the bytes it would have written.
template <int PB16, int RHT = 0, int DEF = 0, int QMODE = 0>
__global__ __launch_bounds__(256) void expand_xt_kernel(const uint32_t* __restrict__ codes, const uint8_t* __restrict__ scales,
                                                        const float* __restrict__ unit_p, uint4* __restrict__ out, int rows,
                                                        int K, int row_tiles, uint32_t sign_mask,
                                                        const uint16_t* __restrict__ center = nullptr,
                                                        const uint32_t* __restrict__ partials = nullptr,
                                                        float* __restrict__ unit_out = nullptr)
{
    typedef float float2_t __attribute__((ext_vector_type(2)));
    static_assert(DEF == 0 || RHT == 0, "deferred scale bytes: unrotated tensors");
    const int lane = threadIdx.x & 63;
    const int kt = K / 32, kgroups = (kt + 7) / 8;
    const int q = lane >> 2, chunk = (lane & 3) ^ xt_swz(q);
    const int64_t nunits = (int64_t)row_tiles * kgroups;
    float unit = 0.0f;
    if constexpr (DEF != 0) {
        unit = tensor_unit_of<QMODE>(fold_partial_maxima(partials));
        if (blockIdx.x == 0 && threadIdx.x == 0) *unit_out = unit;
    } else if constexpr (PB16 != 0) {
        unit = *unit_p;
    }
    const uint16_t* __restrict__ maxima = reinterpret_cast<const uint16_t*>(scales);
    for (int64_t un = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); un < nunits; un += (int64_t)gridDim.x * 4) {
        const int rb_ = (int)(un / kgroups), kg = (int)(un - (int64_t)rb_ * kgroups);
        const int row = rb_ * 16 + q;
        const bool live = row < rows;
        const int kend = min(kt, kg * 8 + 8);
        for (int kb = kg * 8; kb < kend; ++kb) {
            uint4 v = make_uint4(0u, 0u, 0u, 0u);
            if (live) {                                          // lane pairs (l, l ^ 1) share their row: both live or neither
                const int k8 = kb * 4 + chunk;                   // index of the 8-element chunk inside the row
                const uint32_t c = codes[(int64_t)row * (K / 8) + k8];
                uint32_t sb;
                if constexpr (DEF != 0) sb = scale_byte_of<QMODE>(maxima[(int64_t)row * (K / 16) + (k8 >> 1)], unit);
                else sb = scales[(int64_t)row * (K / 16) + (k8 >> 1)];
                if constexpr (RHT != 0) {
                    const float dq = PB16 ? rb(e4m3_value(sb) * unit) : e4m3_value(sb) * 0.00390625f;
                    const float2_t p[4] = {__builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, 1.0f, 0), __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, 1.0f, 1),
                                           __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, 1.0f, 2), __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, 1.0f, 3)};
                    float mine[8], blk[kBlock];
#pragma unroll
                    for (int j = 0; j < 8; ++j) mine[j] = PB16 ? rb(p[j >> 1][j & 1] * dq) : p[j >> 1][j & 1] * dq;
                    const int half = chunk & 1;                  // which half of the block this lane holds
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        // the neighbouring lane's value through DPP (quad_perm 1,0,3,2): no trip through the LDS crossbar
                        const float other = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, mine[j]), 0xB1, 0xf, 0xf, false));
                        blk[j] = half ? other : mine[j];
                        blk[8 + j] = half ? mine[j] : other;
                    }
                    // This lane's half of the rotated block alone, n = 8 half + j: H[k][n] = H[k][j] for k < 8 and
                    // H[k][j] (-1)^half for k >= 8, so the second half of the inputs changes sign with `half` and the sums run
                    // in the order of hadamard16_inverse (a - b and a + (-b) are the same operation).  No array is indexed
                    // by a run-time value: such an array would be moved to LDS.
                    const uint32_t flip = (uint32_t)half << 31;
#pragma unroll
                    for (int k = 8; k < kBlock; ++k) blk[k] = __uint_as_float(__float_as_uint(blk[k]) ^ flip);
                    float o[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        float acc = blk[0];
#pragma unroll
                        for (int k = 1; k < kBlock; ++k) acc = (__builtin_popcount(k & j) & 1) ? acc - blk[k] : acc + blk[k];
                        o[j] = __uint_as_float(__float_as_uint(acc * 0.0625f) ^ (((sign_mask >> (8 * half + j)) & 1u) << 31));
                    }
                    if constexpr (PB16 != 0) {
                        v.x = rb_pair(o[0], o[1]); v.y = rb_pair(o[2], o[3]); v.z = rb_pair(o[4], o[5]); v.w = rb_pair(o[6], o[7]);
                    } else {
                        const half2_t h0 = {(_Float16)o[0], (_Float16)o[1]}, h1 = {(_Float16)o[2], (_Float16)o[3]};
                        const half2_t h2 = {(_Float16)o[4], (_Float16)o[5]}, h3 = {(_Float16)o[6], (_Float16)o[7]};
                        v.x = __builtin_bit_cast(uint32_t, h0); v.y = __builtin_bit_cast(uint32_t, h1);
                        v.z = __builtin_bit_cast(uint32_t, h2); v.w = __builtin_bit_cast(uint32_t, h3);
                    }
                } else if constexpr (PB16 != 0) {
                    const float dq = rb(e4m3_value(sb) * unit);
                    const float2_t p0 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, 1.0f, 0);
                    const float2_t p1 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, 1.0f, 1);
                    const float2_t p2 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, 1.0f, 2);
                    const float2_t p3 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, 1.0f, 3);
                    v.x = rb_pair(p0[0] * dq, p0[1] * dq);
                    v.y = rb_pair(p1[0] * dq, p1[1] * dq);
                    v.z = rb_pair(p2[0] * dq, p2[1] * dq);
                    v.w = rb_pair(p3[0] * dq, p3[1] * dq);
                    if (center) {
                        const uint4 cw = *reinterpret_cast<const uint4*>(center + k8 * 8);
                        v.x = rb_pair(bf16_lo(cw.x) + bf16_lo(v.x), bf16_hi(cw.x) + bf16_hi(v.x));
                        v.y = rb_pair(bf16_lo(cw.y) + bf16_lo(v.y), bf16_hi(cw.y) + bf16_hi(v.y));
                        v.z = rb_pair(bf16_lo(cw.z) + bf16_lo(v.z), bf16_hi(cw.z) + bf16_hi(v.z));
                        v.w = rb_pair(bf16_lo(cw.w) + bf16_lo(v.w), bf16_hi(cw.w) + bf16_hi(v.w));
                    }
                } else {
                    v = expand8(c, scale_pair(sb));
                }
            }
            out[((int64_t)rb_ * kt + kb) * 64 + lane] = v;
        }
    }
}

// Transposing variant: the packed [R, C] tensor (blocks along C) becomes the tiled operand [C, R], the layout a GEMM
// that contracts over R (tokens) reads -- the wgrad operands dY^T and X^T and the dgrad operand W^T of
// src/Metis/Metis/bitlinear.py:502-510.  An output tile (16 operand rows x 32 k) is one block of 16 from each of 32
// source rows: lane l % 32 dequantizes (and, RHT, rotates back) one whole block in registers, the wave turns two
// tiles through LDS and writes them as 2 x 1 KiB of consecutive bytes.  R % 32 == 0.
template <int PB16, int RHT>
__global__ __launch_bounds__(256) void expand_xt_t_kernel(const uint2* __restrict__ codes, const uint8_t* __restrict__ scales,
                                                          const float* __restrict__ unit_p, uint4* __restrict__ out, int R, int C,
                                                          uint32_t sign_mask)
{
    typedef float float2_t __attribute__((ext_vector_type(2)));
    __shared__ __attribute__((aligned(16))) uint16_t turn[4][2][16][40];       // [wave][tile][operand row][k], 80-byte rows
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, half = lane >> 5, sl = lane & 31;
    const int cb_n = C / 16, kt = R / 32, kpairs = (kt + 1) / 2;
    const int64_t nunits = (int64_t)cb_n * kpairs;
    const float unit = PB16 ? *unit_p : 0.0f;
    for (int64_t un = (int64_t)blockIdx.x * 4 + wave; un < nunits; un += (int64_t)gridDim.x * 4) {
        const int cb = (int)(un % cb_n), kp = (int)(un / cb_n);              // consecutive waves: consecutive blocks of a row
        const int kb = kp * 2 + half;
        if (kb < kt) {
            const int r = kb * 32 + sl;
            const uint2 c = codes[(int64_t)r * cb_n + cb];
            const uint32_t sb = scales[(int64_t)r * cb_n + cb];
            const float dq = PB16 ? rb(e4m3_value(sb) * unit) : e4m3_value(sb) * 0.00390625f;
            float blk[kBlock];
            const float2_t p[8] = {__builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.x, 1.0f, 0), __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.x, 1.0f, 1),
                                   __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.x, 1.0f, 2), __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.x, 1.0f, 3),
                                   __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.y, 1.0f, 0), __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.y, 1.0f, 1),
                                   __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.y, 1.0f, 2), __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.y, 1.0f, 3)};
#pragma unroll
            for (int j = 0; j < 8; ++j) { blk[2 * j] = p[j][0] * dq; blk[2 * j + 1] = p[j][1] * dq; }
            if constexpr (PB16 != 0) {
#pragma unroll
                for (int j = 0; j < kBlock; ++j) blk[j] = rb(blk[j]);
            }
            if constexpr (RHT != 0) hadamard16_inverse(blk, sign_mask);
#pragma unroll
            for (int j = 0; j < kBlock; ++j)
                turn[wave][half][j][sl] = PB16 ? (uint16_t)bf16_bits(blk[j]) : __builtin_bit_cast(uint16_t, (_Float16)blk[j]);
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);                      // LDS writes of this wave are done (lgkmcnt 0)
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int tl = 0; tl < 2; ++tl) {
            if (kp * 2 + tl < kt) {
                const int q = lane >> 2, chunk = (lane & 3) ^ xt_swz(q);
                const uint4 v = *reinterpret_cast<const uint4*>(&turn[wave][tl][q][chunk * 8]);
                out[((int64_t)cb * kt + kp * 2 + tl) * 64 + lane] = v;
            }
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_wave_barrier();
    }
}

// A dense [R, K] tensor (bf16 or binary32, row stride ld) in the same tiled layout: binary16 (PB16 = 0: one rounding of
// each value; no prescale, so the caller passes 2^-8 as this operand's unit to cancel the 2^8 the GEMM applies for an
// exact expansion) or bf16 (PB16 = 1).  col_scale (optional, bf16 [K]) multiplies column
// k first, rounded to the tensor's dtype as `weight * s.unsqueeze(0)` rounds (src/Metis/Metis/bitlinear.py:727).
// The dense operand of the merged rollout forward (705-751): U diag(s) and the merged weight itself.
template <int PB16, int F32>
__global__ __launch_bounds__(256) void dense_xt_kernel(const void* __restrict__ xv, int64_t ld, const uint16_t* __restrict__ col_scale,
                                                       uint4* __restrict__ out, int rows, int K, int row_tiles)
{
    const int lane = threadIdx.x & 63;
    const int kt = K / 32;
    const int q = lane >> 2, chunk = (lane & 3) ^ xt_swz(q);
    const int64_t ntiles = (int64_t)row_tiles * kt;
    for (int64_t tile = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); tile < ntiles; tile += (int64_t)gridDim.x * 4) {
        const int rb_ = (int)(tile / kt), kb = (int)(tile - (int64_t)rb_ * kt);
        const int row = rb_ * 16 + q, k0 = kb * 32 + chunk * 8;
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        if (row < rows) {
            float f[8];
            if (F32) {
                const float4* p = reinterpret_cast<const float4*>(static_cast<const float*>(xv) + (int64_t)row * ld + k0);
                const float4 a = p[0], b = p[1];
                f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
            } else {
                const uint4 w = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(xv) + (int64_t)row * ld + k0);
                f[0] = bf16_lo(w.x); f[1] = bf16_hi(w.x); f[2] = bf16_lo(w.y); f[3] = bf16_hi(w.y);
                f[4] = bf16_lo(w.z); f[5] = bf16_hi(w.z); f[6] = bf16_lo(w.w); f[7] = bf16_hi(w.w);
            }
            if (col_scale) {
                const uint4 w = *reinterpret_cast<const uint4*>(col_scale + k0);
                const float sc[8] = {bf16_lo(w.x), bf16_hi(w.x), bf16_lo(w.y), bf16_hi(w.y), bf16_lo(w.z), bf16_hi(w.z), bf16_lo(w.w), bf16_hi(w.w)};
#pragma unroll
                for (int j = 0; j < 8; ++j) f[j] = F32 ? f[j] * sc[j] : rb(f[j] * sc[j]);
            }
            if constexpr (PB16 != 0) {
                v.x = rb_pair(f[0], f[1]); v.y = rb_pair(f[2], f[3]); v.z = rb_pair(f[4], f[5]); v.w = rb_pair(f[6], f[7]);
            } else {
                const half2_t h0 = {(_Float16)f[0], (_Float16)f[1]}, h1 = {(_Float16)f[2], (_Float16)f[3]};
                const half2_t h2 = {(_Float16)f[4], (_Float16)f[5]}, h3 = {(_Float16)f[6], (_Float16)f[7]};
                v.x = __builtin_bit_cast(uint32_t, h0); v.y = __builtin_bit_cast(uint32_t, h1);
                v.z = __builtin_bit_cast(uint32_t, h2); v.w = __builtin_bit_cast(uint32_t, h3);
            }
        }
        out[tile * 64 + lane] = v;
    }
}

int dense_xt(const void* x, int64_t rows, int64_t cols, int64_t ld, int dtype, const void* col_scale, int mode, void* out, hipStream_t st)
{
    if (rows < 0 || cols < 0 || ld < cols) return METIS_E_ARG;
    if (mode == METIS_MODE_P32_F32) mode = METIS_MODE_P32;
    if (mode != METIS_MODE_P32 && mode != METIS_MODE_PB16) return METIS_E_ARG;
    if (dtype != METIS_DTYPE_BF16 && dtype != METIS_DTYPE_F32) return METIS_E_ARG;
    if (cols % 32) return METIS_E_SHAPE;
    if (rows > INT32_MAX - 16 || cols > INT32_MAX) return METIS_E_ARG;
    if (rows == 0 || cols == 0) return METIS_OK;
    const int al = dtype == METIS_DTYPE_F32 ? 4 : 8;
    if (!x || !out || (ld % al) || ((uintptr_t)x % 16) || ((uintptr_t)out % 16) || ((uintptr_t)col_scale % 16)) return METIS_E_ARG;
    const int row_tiles = (int)((rows + 15) / 16);
    const int64_t ntiles = (int64_t)row_tiles * (cols / 32);
    int64_t g = (ntiles + 3) / 4;
    const int64_t cap = (int64_t)device_cus() * 16;
    if (g > cap) g = cap;
#define METIS_DX(P, F) hipLaunchKernelGGL((dense_xt_kernel<P, F>), dim3((unsigned)g), dim3(256), 0, st, x, ld, (const uint16_t*)col_scale, \
                                          (uint4*)out, (int)rows, (int)cols, row_tiles)
    if (mode == METIS_MODE_PB16) { if (dtype == METIS_DTYPE_F32) METIS_DX(1, 1); else METIS_DX(1, 0); }
    else { if (dtype == METIS_DTYPE_F32) METIS_DX(0, 1); else METIS_DX(0, 0); }
#undef METIS_DX
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

size_t expand_xt_bytes(int64_t rows, int64_t cols)
{
    if (rows <= 0 || cols <= 0) return 0;
    return (size_t)((rows + 15) / 16) * 16 * (size_t)cols * 2;
}

int expand_xt(const void* codes, const void* scales, const float* unit, int64_t rows, int64_t cols, int mode, void* out,
              hipStream_t st, int rht, uint32_t sign_mask, const void* center)
{
    if (rows < 0 || cols < 0 || sign_mask > 0xffffu) return METIS_E_ARG;
    if (center && (mode != METIS_MODE_PB16 || rht || ((uintptr_t)center % 16))) return METIS_E_ARG;   // a centre belongs to bf16 arithmetic
    if (mode == METIS_MODE_P32_F32) mode = METIS_MODE_P32;
    if (mode != METIS_MODE_P32 && mode != METIS_MODE_PB16) return METIS_E_ARG;
    if (cols % kBlock) return METIS_E_SHAPE;
    if (cols % 32 || rows > INT32_MAX - 16 || cols > INT32_MAX) return METIS_E_ARG;
    if (rows == 0 || cols == 0) return METIS_OK;
    if (!codes || !scales || !out || ((uintptr_t)codes % 4) || ((uintptr_t)out % 16)) return METIS_E_ARG;
    if (mode == METIS_MODE_PB16 && !unit) return METIS_E_ARG;
    const int row_tiles = (int)((rows + 15) / 16);
    const int64_t units = (int64_t)row_tiles * ((cols / 32 + 7) / 8);
    int64_t g = (units + 3) / 4;
    const int64_t cap = (int64_t)device_cus() * 16;
    if (g > cap) g = cap;
#define METIS_EX(P, R) hipLaunchKernelGGL((expand_xt_kernel<P, R>), dim3((unsigned)g), dim3(256), 0, st, (const uint32_t*)codes, \
                                          (const uint8_t*)scales, unit, (uint4*)out, (int)rows, (int)cols, row_tiles, sign_mask)
    if (center) {
        hipLaunchKernelGGL((expand_xt_kernel<1, 0>), dim3((unsigned)g), dim3(256), 0, st, (const uint32_t*)codes, (const uint8_t*)scales,
                           unit, (uint4*)out, (int)rows, (int)cols, row_tiles, sign_mask, (const uint16_t*)center);
        return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
    }
    if (mode == METIS_MODE_PB16) { if (rht) METIS_EX(1, 1); else METIS_EX(1, 0); }
    else { if (rht) METIS_EX(0, 1); else METIS_EX(0, 0); }
#undef METIS_EX
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

int expand_xt_deferred(const void* codes, const void* deferred, int64_t rows, int64_t cols, int qmode, int mode, const void* center,
                       float* unit_out, void* out, hipStream_t st)
{
    if (rows < 0 || cols < 0) return METIS_E_ARG;
    if (center && (mode != METIS_MODE_PB16 || ((uintptr_t)center % 16))) return METIS_E_ARG;   // a centre belongs to bf16 arithmetic
    if (mode == METIS_MODE_P32_F32) mode = METIS_MODE_P32;
    if ((mode != METIS_MODE_P32 && mode != METIS_MODE_PB16) || (qmode != METIS_MODE_P32 && qmode != METIS_MODE_PB16)) return METIS_E_ARG;
    if (cols % kBlock) return METIS_E_SHAPE;
    if (cols % 32 || rows > INT32_MAX - 16 || cols > INT32_MAX) return METIS_E_ARG;
    if (rows == 0 || cols == 0) return METIS_OK;
    if (!codes || !unit_out || !out || ((uintptr_t)codes % 4) || ((uintptr_t)out % 16)) return METIS_E_ARG;
    Workspace ws;
    if (const int rc = carve_deferred(const_cast<void*>(deferred), deferred_bytes(rows, cols), rows, cols, &ws)) return rc;
    const int row_tiles = (int)((rows + 15) / 16);
    const int64_t units = (int64_t)row_tiles * ((cols / 32 + 7) / 8);
    int64_t g = (units + 3) / 4;
    const int64_t cap = (int64_t)device_cus() * 16;
    if (g > cap) g = cap;
#define METIS_EXD(P, Q) hipLaunchKernelGGL((expand_xt_kernel<P, 0, 1, Q>), dim3((unsigned)g), dim3(256), 0, st, (const uint32_t*)codes, \
                                           (const uint8_t*)ws.amax, nullptr, (uint4*)out, (int)rows, (int)cols, row_tiles, 0u, \
                                           (const uint16_t*)center, (const uint32_t*)ws.gmax, unit_out)
    if (mode == METIS_MODE_PB16) { if (qmode) METIS_EXD(1, 1); else METIS_EXD(1, 0); }
    else { if (qmode) METIS_EXD(0, 1); else METIS_EXD(0, 0); }
#undef METIS_EXD
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

int expand_xt_transposed(const void* codes, const void* scales, const float* unit, int64_t rows, int64_t cols, int mode, void* out,
                         hipStream_t st, int rht, uint32_t sign_mask)
{
    if (rows < 0 || cols < 0 || sign_mask > 0xffffu) return METIS_E_ARG;
    if (mode == METIS_MODE_P32_F32) mode = METIS_MODE_P32;
    if (mode != METIS_MODE_P32 && mode != METIS_MODE_PB16) return METIS_E_ARG;
    if (cols % kBlock || rows % 32) return METIS_E_SHAPE;
    if (rows > INT32_MAX - 32 || cols > INT32_MAX) return METIS_E_ARG;
    if (rows == 0 || cols == 0) return METIS_OK;
    if (!codes || !scales || !out || ((uintptr_t)codes % 8) || ((uintptr_t)out % 16)) return METIS_E_ARG;
    if (mode == METIS_MODE_PB16 && !unit) return METIS_E_ARG;
    const int64_t units = (cols / 16) * ((rows / 32 + 1) / 2);
    int64_t g = (units + 3) / 4;
    const int64_t cap = (int64_t)device_cus() * 16;
    if (g > cap) g = cap;
#define METIS_EXT(P, R) hipLaunchKernelGGL((expand_xt_t_kernel<P, R>), dim3((unsigned)g), dim3(256), 0, st, (const uint2*)codes, \
                                           (const uint8_t*)scales, unit, (uint4*)out, (int)rows, (int)cols, sign_mask)
    if (mode == METIS_MODE_PB16) { if (rht) METIS_EXT(1, 1); else METIS_EXT(1, 0); }
    else { if (rht) METIS_EXT(0, 1); else METIS_EXT(0, 0); }
#undef METIS_EXT
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

// ---------------------------------------------------------------------------------------------
// The GEMM.  256 x 256 per workgroup, eight waves (2 x 4) of 128 x 64, two per SIMD.
// A stage is 32 k of the A|B tile: 32 KiB = 32 operand tiles, one direct load each.  Three slots form a ring
// (96 KiB).  Iteration s (stage s in slot s % 3):
//     read fragments (s, k 16..31)            | MFMAs on fragments (s, k 0..15)
//     wait: own fragment reads done, own loads of stage s+1 landed;  BARRIER
//     read fragments (s+1, k 0..15); loads of stage s+3 into slot s % 3, spread between the MFMAs on fragments
//     (s, k 16..31): every wave holds what it needs of stage s in registers by then
// so a stage's loads have two iterations to arrive and the waits never drain the queue.
// Measured at 8192 x 14336 x 4096 before these choices were fixed: rings of 3, 4 and 5 slots within 1 % of each
// other (latency is covered); loads spread between the MFMAs 1-2 % faster than issued in one burst; two stages
// per barrier 3 % slower; four waves of 128 x 128 (a third less LDS read traffic, one wave per SIMD) 17 % slower.
//
// PB16: operands are the reference's bf16 dequantized values (bf16 MFMA, no unit factor), and the epilogue
// rounds where the reference's all-bf16 evaluation rounds: the residual product to bf16 (its bf16 matmul), the
// bias added in bf16, then the low-rank term and the final rounding (bitlinear.py:435-438 under compute_dtype =
// bfloat16, src/grpo/grpo.py:204-205).
// SPLIT: as in gemm_nvfp4_large_kernel -- tiles nfull .. total-1 have nsplit workgroups each, every one contracting
// its own range of stages into a binary32 partial tile in ws (accumulator-register order) for
// gemm_splitk_reduce_kernel, which also forms the low-rank term of the tile and adds the bias.  Exact mode: units
// applied; PB16: the reduction kernel rounds the sum and adds the bias in bf16, as the reference's bf16 forward does.
// ---------------------------------------------------------------------------------------------
constexpr int XT_STAGE = 32 * 1024, XT_NS = 3;
// Beyond the ring: the first two 32-column steps of the rank-r factors T | U of the tile (512 rows x 32 columns each, in the
// operand tile format), requested by direct loads before the first operand stage, so that the low-rank extension at the
// end of the tile finds them in LDS instead of waiting for two dependent memory round trips.
constexpr int XT_LR_STEPS = 2, XT_LDS = (XT_NS + XT_LR_STEPS) * XT_STAGE;     // 160 KiB: all of a compute unit's LDS

__host__ __device__ constexpr int waitcnt_imm(int vm, int lgkm)
{
    return (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | ((lgkm & 15) << 8);
}
#define METIS_WAIT(VM, LGKM) __builtin_amdgcn_s_waitcnt(waitcnt_imm(VM, LGKM))

template <int OUT_F32, int PB16, int SPLIT>
__global__ __launch_bounds__(512, 1) void gemm_xt_kernel(
    const uint8_t* __restrict__ a_xt, const float* __restrict__ a_unit, const uint8_t* __restrict__ b_xt,
    const float* __restrict__ b_unit, int M, int N, int K, const uint16_t* __restrict__ t, const uint16_t* __restrict__ u,
    int r, const uint16_t* __restrict__ bias, void* __restrict__ out, int tiles_m, int tiles_n, int bias_f32,
    float* __restrict__ ws, int nsplit, int nfull)
{
    extern __shared__ __attribute__((aligned(1024))) uint8_t xlds[];
    constexpr int TM = 4, TN = 2, WTN = 64, NWAVES = 8, NTHREADS = 512, NS = XT_NS;
    constexpr int LPW = 32 / NWAVES;                            // direct loads per wave per stage
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / 4, wn = wave % 4;

    // ---- tile assignment: contiguous range per XCD, groups of four tile rows (see tile_origin).  SPLIT: the first
    //      nfull tiles (a multiple of 8) run unsplit, every XCD its share of them first; the rest have nsplit workgroups each.
    const int total = tiles_m * tiles_n;
    int logical, split = 0;
    bool partial = false;
    if constexpr (SPLIT != 0) {
        const int xcd = blockIdx.x & 7, li = blockIdx.x >> 3, full_x = nfull >> 3;
        if (li < full_x) {
            logical = xcd * full_x + li;
        } else {
            const int tail = total - nfull, tail_all = tail * nsplit, per_xcd = (tail_all + 7) / 8;
            const int j = xcd * per_xcd + (li - full_x);
            if (li - full_x >= per_xcd || j >= tail_all) return;
            split = j / tail;                                    // consecutive workgroups of an XCD share a K range
            logical = nfull + j % tail;
            partial = true;
        }
    } else {
        const int per_xcd = (total + 7) / 8;
        logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
        if (logical >= total) return;
    }
    int m0, n0;
    tile_origin(logical, tiles_m, tiles_n, m0, n0);
    const int kt = K / 32;
    const int step_begin = partial ? (int)((int64_t)split * kt / nsplit) : 0;
    const int steps = (partial ? (int)((int64_t)(split + 1) * kt / nsplit) : kt) - step_begin;   // >= 1: the host never asks for more splits than stages

    float16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    // ---- direct loads: instruction j of wave w copies operand tile j * 8 + w of the stage (0..15 A, 16..31 B).
    // Written as assembly: the compiler orders every later LDS read behind ALL outstanding direct loads (it cannot
    // tell the ring slots apart), which would drain the queue each iteration; the waits are placed by hand instead.
    const int a_rt = (M + 15) / 16, b_rt = (N + 15) / 16;
    const uint8_t* src[LPW];                                    // wave-uniform: the tile row at the first stage of this workgroup
#pragma unroll
    for (int j = 0; j < LPW; ++j) {
        const int ot = j * NWAVES + wave;
        const bool is_a = ot < 16;
        const int rt = is_a ? min(m0 / 16 + ot, a_rt - 1) : min(n0 / 16 + ot - 16, b_rt - 1);
        src[j] = (is_a ? a_xt : b_xt) + ((int64_t)rt * kt + step_begin) * 1024;
    }
    const uint32_t lane16 = lane * 16;
    auto issue_one = [&](int slot, int it, int j) {
        const uint8_t* g = src[j] + (int64_t)it * 1024;
        const uint32_t dst = (uint32_t)(slot * XT_STAGE + (j * NWAVES + wave) * 1024);   // LDS byte address of the tile
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :: "v"(lane16), "s"(g), "s"(dst) : "memory");
    };

    // ---- rank-r factors ahead of everything else: instruction j of wave w gathers the 16 rows x 32 columns piece
    //      j * 8 + w of T | U (0..15 rows of T, 16..31 rows of U) for step p, every lane its 16 bytes, into the slot
    //      order of an operand tile.  They are the oldest loads of the wave: whatever wait covers an operand stage covers them.
    // (Kernels with split tiles keep the staged form for all steps: their register budget has no room for both.)
    const int lr_ahead = (SPLIT == 0 && t != nullptr) ? min(r / 32, XT_LR_STEPS) : 0;
    if constexpr (SPLIT == 0) {
        const int q = lane >> 2, chunk = (lane & 3) ^ xt_swz(q);
        for (int p = 0; p < lr_ahead; ++p) {
#pragma unroll
            for (int j = 0; j < LPW; ++j) {
                const int ot = j * NWAVES + wave;
                const bool is_a = ot < 16;
                const int64_t row = is_a ? min(m0 + ot * 16 + q, M - 1) : min(n0 + (ot - 16) * 16 + q, N - 1);
                const uint16_t* g = (is_a ? t : u) + row * r + p * 32 + chunk * 8;
                const uint32_t dst = (uint32_t)((NS + p) * XT_STAGE + ot * 1024);
                asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(g), "s"(dst) : "memory");
            }
        }
    }

    // ---- fragment addressing: lane -> row lr of a 32-row MFMA tile, k half hi; chunk = 2 * ks + hi.
    // ks = 1 flips bit 1 of the chunk index, which flips bit 1 of the slot: byte offset ^ 32.
    const int lr = lane & 31, hi = lane >> 5;
    const int lane_off = (lr >> 4) * 1024 + (lr & 15) * 64 + ((hi ^ xt_swz(lr & 15)) * 16);
    const int a_off[2] = {wm * 8 * 1024 + lane_off, wm * 8 * 1024 + (lane_off ^ 32)};
    const int b_off[2] = {(16 + wn * (WTN / 16)) * 1024 + lane_off, (16 + wn * (WTN / 16)) * 1024 + (lane_off ^ 32)};
    uint4 fa[2][TM], fb[2][TN];                                 // 8 binary16 / bf16 values each
    auto load_frags = [&](int slot, int ks) {
        const int x = slot * XT_STAGE;
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[ks][i] = *reinterpret_cast<const uint4*>(xlds + (a_off[ks] + x) + i * 2048);
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[ks][j] = *reinterpret_cast<const uint4*>(xlds + (b_off[ks] + x) + j * 2048);
    };
    auto mfma_one = [&](int fbuf, int i, int j) {
        if constexpr (PB16 != 0)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, fb[fbuf][j]),
                                                                __builtin_bit_cast(bf16x8_t, fa[fbuf][i]), acc[i][j], 0, 0, 0);
        else
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, fb[fbuf][j]),
                                                               __builtin_bit_cast(half8_t, fa[fbuf][i]), acc[i][j], 0, 0, 0);
    };
    auto mfmas = [&](int fbuf) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) mfma_one(fbuf, i, j);
    };
    constexpr int NM = TM * TN, NF = TM + TN;

    // prologue: fill the ring
#pragma unroll
    for (int p = 0; p < NS; ++p)
        if (p < steps) {
#pragma unroll
            for (int j = 0; j < LPW; ++j) issue_one(p, p, j);
        }
    if (steps >= NS) METIS_WAIT((NS - 1) * LPW, 15);
    else METIS_WAIT(0, 15);
    __syncthreads();
    load_frags(0, 0);

    int s = 0, slot = 0;
    // steady state: the stage NS ahead exists, so every wait allows NS-2 stages in flight
    for (; s + NS < steps; ++s) {
        const int nslot = slot + 1 == NS ? 0 : slot + 1;
        load_frags(slot, 1);
        mfmas(0);
        sched_substep<NM, 0, NF, 0>();
        METIS_WAIT((NS - 2) * LPW, 0);                          // own loads of stage s+1 landed, own fragment reads of stage s done
        __syncthreads();
        load_frags(nslot, 0);
        constexpr int PER = NM / LPW;                           // one direct load every PER MFMAs
#pragma unroll
        for (int m = 0; m < NM; ++m) {
            if (m % PER == 0) issue_one(slot, s + NS, m / PER);
            mfma_one(1, m / TN, m % TN);
        }
        slot = nslot;
    }
    // drain: nothing left to issue; the loads still in flight are at most NS-1 stages
    for (; s < steps; ++s) {
        const int nslot = slot + 1 == NS ? 0 : slot + 1;
        load_frags(slot, 1);
        mfmas(0);
        sched_substep<NM, 0, NF, 0>();
        METIS_WAIT(0, 0);
        __syncthreads();
        if (s + 1 < steps) load_frags(nslot, 0);
        mfmas(1);
        sched_substep<NM, 0, NF, 0>();
        slot = nslot;
    }
    __syncthreads();                                            // the ring is free for the epilogue

    float* wt = nullptr;
    if (SPLIT != 0 && partial) wt = ws + (size_t)(split * (total - nfull) + (logical - nfull)) * (L_BM * L_BN) + tid * 4;
    auto store_partial = [&](float* dst, bool with_bias) {      // accumulator-register order, 1 KiB per store instruction
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int n = n0 + wn * WTN + j * 32 + 8 * g + 4 * hi;
                    float v[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        v[e] = acc[i][j][4 * g + e];
                        if (with_bias && bias) v[e] += bias_value(bias, bias_f32, min(n + e, N - 1));
                    }
                    *reinterpret_cast<float4*>(dst + ((i * TN + j) * 4 + g) * (NTHREADS * 4)) = make_float4(v[0], v[1], v[2], v[3]);
                }
    };

    if constexpr (PB16 != 0) {
        if (SPLIT != 0 && partial) {
            store_partial(wt, false);                           // the residual product of this K range; the reduction kernel
            return;                                             // rounds the sum and adds bias and low-rank term
        } else {
            // the reference's bf16 matmul result, then its bf16 bias add
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        float v = rb(acc[i][j][e]);
                        if (bias) v = rb(v + bias_value(bias, bias_f32, min(n0 + wn * WTN + j * 32 + 8 * (e >> 2) + 4 * hi + (e & 3), N - 1)));
                        acc[i][j][e] = v;
                    }
            bias = nullptr;
        }
    } else {
        // tensor units (and the 2^8 * 2^8 of the scale placement)
        const float us = (*a_unit) * (*b_unit) * 65536.0f;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] *= us;
        if (SPLIT != 0 && partial) {
            store_partial(wt, false);                           // this split's share; low-rank term and bias wait for the sum
            return;
        }
    }

    // ---- bf16 low-rank extension: the steps that were requested ahead are one more operand stage each
    if constexpr (SPLIT == 0)
    for (int p = 0; p < lr_ahead; ++p) {
        const int x = (NS + p) * XT_STAGE;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            bf16x8_t ga[TM], gb[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) ga[i] = *reinterpret_cast<const bf16x8_t*>(xlds + (a_off[ks] + x) + i * 2048);
#pragma unroll
            for (int j = 0; j < TN; ++j) gb[j] = *reinterpret_cast<const bf16x8_t*>(xlds + (b_off[ks] + x) + j * 2048);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gb[j], ga[i], acc[i][j], 0, 0, 0);
        }
    }
    // ---- further steps (r > 64): 32 columns of T / U per step, staged in rows of 144 bytes
    uint16_t* plds = reinterpret_cast<uint16_t*>(xlds);
    const int frag_off = lr * L_STRIDE + hi * 8;
    for (int j0 = lr_ahead * 32; j0 < r; j0 += 32) {
        {
            const int trow = tid;                               // 512 threads, 512 rows of the T|U tile
            const bool is_a = trow < L_BM;
            const int64_t grow = is_a ? min(m0 + trow, M - 1) : min(n0 + trow - L_BM, N - 1);
            const uint4* sp = reinterpret_cast<const uint4*>((is_a ? t : u) + grow * r + j0);
            uint4* dp = reinterpret_cast<uint4*>(plds + trow * L_STRIDE);
#pragma unroll
            for (int c = 0; c < 4; ++c) dp[c] = sp[c];
        }
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            bf16x8_t ga[TM], gb[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) ga[i] = *reinterpret_cast<const bf16x8_t*>(plds + (wm * 128 + i * 32) * L_STRIDE + frag_off + ks * 16);
#pragma unroll
            for (int j = 0; j < TN; ++j) gb[j] = *reinterpret_cast<const bf16x8_t*>(plds + (L_BM + wn * WTN + j * 32) * L_STRIDE + frag_off + ks * 16);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gb[j], ga[i], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    if constexpr (PB16 != 0 && OUT_F32 != 0) {                  // a binary32 output buffer still holds bf16 values in this mode
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] = rb(acc[i][j][e]);
    }

    // ---- epilogue.  acc[i][j][e] of lane l: m = 32 i + l % 32, n = 32 j + 8 (e / 4) + 4 (l / 32) + e % 4 in the wave tile.
    if constexpr (!OUT_F32) {
        if ((N & 7) == 0) {
            // bf16: each wave transposes its tile through its own slice of LDS, 64 rows at a time, so that a store
            // instruction writes 8 rows x 128 contiguous bytes
            constexpr int CROW = WTN + 8;                       // halves per staged row: 144 bytes
            constexpr int LPR = WTN / 8, RPI = 64 / LPR;        // lanes per row, rows per store instruction
            uint16_t* cw = plds + wave * (64 * CROW);
            const int rsub = lane / LPR, chunk = lane % LPR;
            const int n = n0 + wn * WTN + chunk * 8;
#pragma unroll
            for (int pass = 0; pass < 2; ++pass) {
#pragma unroll
                for (int ii = 0; ii < 2; ++ii)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
                            const int nl = j * 32 + 8 * g + 4 * hi;
                            float v[4];
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                v[e] = acc[pass * 2 + ii][j][4 * g + e];
                                if (bias) v[e] += bias_value(bias, bias_f32, min(n0 + wn * WTN + nl + e, N - 1));
                            }
                            uint2 w;
                            w.x = bf16_bits(v[0]) | (bf16_bits(v[1]) << 16);
                            w.y = bf16_bits(v[2]) | (bf16_bits(v[3]) << 16);
                            *reinterpret_cast<uint2*>(cw + (ii * 32 + lr) * CROW + nl) = w;
                        }
                __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, 0));   // the wave reads back what it wrote itself
#pragma unroll
                for (int it = 0; it < 64 / RPI; ++it) {
                    const int ml = it * RPI + rsub;
                    const int m = m0 + wm * 128 + pass * 64 + ml;
                    const uint4 w = *reinterpret_cast<const uint4*>(cw + ml * CROW + chunk * 8);
                    if (m < M && n < N) *reinterpret_cast<uint4*>((uint16_t*)out + (int64_t)m * N + n) = w;
                }
            }
            return;
        }
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = m0 + wm * 128 + i * 32 + lr;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = n0 + wn * WTN + j * 32 + 8 * g + 4 * hi;
                if (n >= N) continue;                            // N % 4 == 0
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[e] = acc[i][j][4 * g + e];
                    if (bias) v[e] += bias_value(bias, bias_f32, n + e);
                }
                if (OUT_F32) {
                    *reinterpret_cast<float4*>((float*)out + (int64_t)m * N + n) = make_float4(v[0], v[1], v[2], v[3]);
                } else {
                    uint2 w;
                    w.x = bf16_bits(v[0]) | (bf16_bits(v[1]) << 16);
                    w.y = bf16_bits(v[2]) | (bf16_bits(v[3]) << 16);
                    *reinterpret_cast<uint2*>((uint16_t*)out + (int64_t)m * N + n) = w;
                }
            }
        }
    }
}

// K splits of the pipelined kernel: the plan of the packed kernel (same tiles), with a stage of 32 k as the unit.
static SplitPlan xt_split_plan(int64_t M, int64_t N, int64_t K)
{
    SplitPlan p = split_plan(M, N, K);                          // needs K % 64 == 0, M and N >= 256
    if (p.nsplit > K / 32) p.nsplit = (int)(K / 32);
    return p.nsplit < 2 ? SplitPlan{1, 0} : p;
}

size_t gemm_xt_workspace_bytes(int64_t M, int64_t N, int64_t K, int mode)
{
    if (M <= 0 || N <= 0 || K <= 0 || K % 32) return 0;
    const SplitPlan p = xt_split_plan(M, N, K);
    if (p.nsplit <= 1) return 0;
    const int64_t tiles = ((M + L_BM - 1) / L_BM) * ((N + L_BN - 1) / L_BN);
    const int slots = p.nsplit + (mode == METIS_MODE_PB16 ? 1 : 0);
    return (size_t)slots * (size_t)(tiles - p.nfull) * L_BM * L_BN * sizeof(float);
}

template <int OUT_F32, int PB16, int SPLIT>
static int launch_xt(const void* a_xt, const float* a_unit, const void* b_xt, const float* b_unit, int64_t M, int64_t N, int64_t K,
                     const void* t, const void* u, int64_t r, const void* bias, int bias_f32, void* out, hipStream_t st, float* ws,
                     int nsplit, int nfull)
{
    static bool attr_set[64] = {};
    const void* fn = (const void*)gemm_xt_kernel<OUT_F32, PB16, SPLIT>;
    const size_t lds_bytes = (size_t)XT_LDS;
    if (const int rc = allow_dynamic_lds(fn, lds_bytes, attr_set)) return rc;
    const int tiles_m = (int)((M + L_BM - 1) / L_BM), tiles_n = (int)((N + L_BN - 1) / L_BN);
    const int total = tiles_m * tiles_n;
    const unsigned grid_x = SPLIT ? 8u * (unsigned)(nfull / 8 + ((total - nfull) * nsplit + 7) / 8) : (unsigned)(((total + 7) / 8) * 8);
    const uint8_t *ae = (const uint8_t*)a_xt, *be = (const uint8_t*)b_xt;
    const uint16_t *tp = (const uint16_t*)t, *up = (const uint16_t*)u, *bp = (const uint16_t*)bias;
    int Mi = (int)M, Ni = (int)N, Ki = (int)K, ri = (int)r, tmi = tiles_m, tni = tiles_n;
    void* args[] = {&ae, &a_unit, &be, &b_unit, &Mi, &Ni, &Ki, &tp, &up, &ri, &bp, &out, &tmi, &tni, &bias_f32, &ws, &nsplit, &nfull};
    if (hipLaunchKernel(fn, dim3(grid_x), dim3(512), args, lds_bytes, st) != hipSuccess) {
        (void)hipGetLastError();
        return METIS_E_LAUNCH;
    }
    if (SPLIT) {
        const dim3 rgrid((unsigned)(total - nfull) * 32u);
        hipLaunchKernelGGL((gemm_splitk_reduce_kernel<OUT_F32, PB16>), rgrid, dim3(64), 0, st, (const float*)ws, nsplit, Mi, Ni, tmi, tni, out,
                           nfull, bp, bias_f32, tp, up, ri);
        if (hipGetLastError() != hipSuccess) return METIS_E_LAUNCH;
    }
    return METIS_OK;
}

int gemm_xt(const void* a_xt, const float* a_unit, const void* b_xt, const float* b_unit, int64_t M, int64_t N, int64_t K,
            const void* t, const void* u, int64_t r, const void* bias, int bias_f32, void* out, int out_dtype, int mode,
            void* workspace, size_t workspace_bytes, hipStream_t st)
{
    if (M < 0 || N < 0 || K < 0 || r < 0) return METIS_E_ARG;
    if (out_dtype != METIS_DTYPE_BF16 && out_dtype != METIS_DTYPE_F32) return METIS_E_ARG;
    if (mode == METIS_MODE_P32_F32) mode = METIS_MODE_P32;
    if (mode != METIS_MODE_P32 && mode != METIS_MODE_PB16) return METIS_E_ARG;
    if (K % kBlock) return METIS_E_SHAPE;
    if (K % 32 || K == 0 || N % 4 || r % 32 || (r > 0 && (!t || !u))) return METIS_E_ARG;
    if (M > INT32_MAX - 256 || N > INT32_MAX - 256 || K > INT32_MAX) return METIS_E_ARG;
    if (M == 0 || N == 0) return METIS_OK;
    if (!a_xt || !b_xt || !out || (mode == METIS_MODE_P32 && (!a_unit || !b_unit))) return METIS_E_ARG;
    if (((uintptr_t)a_xt % 16) || ((uintptr_t)b_xt % 16) || ((uintptr_t)out % 16) || ((uintptr_t)t % 16) || ((uintptr_t)u % 16) ||
        ((uintptr_t)bias % (bias_f32 ? 4 : 2)))
        return METIS_E_ARG;
    SplitPlan plan = {1, 0};
    if (workspace) {
        plan = xt_split_plan(M, N, K);
        if (plan.nsplit > 1 && (((uintptr_t)workspace % 16) || workspace_bytes < gemm_xt_workspace_bytes(M, N, K, mode))) return METIS_E_WORKSPACE;
    }
    const int f32 = out_dtype == METIS_DTYPE_F32, pb = mode == METIS_MODE_PB16, sp = plan.nsplit > 1;
#define METIS_XT(F, P, S) launch_xt<F, P, S>(a_xt, a_unit, b_xt, b_unit, M, N, K, t, u, r, bias, bias_f32, out, st, (float*)workspace, \
                                            plan.nsplit, plan.nfull)
    switch (f32 * 4 + pb * 2 + sp) {
        case 0: return METIS_XT(0, 0, 0);
        case 1: return METIS_XT(0, 0, 1);
        case 2: return METIS_XT(0, 1, 0);
        case 3: return METIS_XT(0, 1, 1);
        case 4: return METIS_XT(1, 0, 0);
        case 5: return METIS_XT(1, 0, 1);
        case 6: return METIS_XT(1, 1, 0);
        default: return METIS_XT(1, 1, 1);
    }
#undef METIS_XT
}

}  // namespace metis
