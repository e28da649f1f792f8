// Block-scaled NVFP4 GEMM with a bf16 low-rank extension, for gfx950 MFMA.
//
//   out[M,N] = ua*ub * sum_k deq(A)[m,k] deq(B)[n,k]  +  sum_j T[m,j] U[n,j]  +  bias[n]
//
// Replaces torch.matmul(input_, quantized_weight.T) (+ bias) of LinearLowbitFunction.forward
// (src/Metis/Metis/bitlinear.py:435-438), the two backward matmuls (502-508) and the sum of the
// rank-r and residual branches of BitLinear.forward (752-760).
//
// Numerics: an E2M1 value times an E4M3 value has at most 5 significant bits and fits the
// exponent range of binary16, so each packed operand is expanded EXACTLY to binary16 in LDS
// (hardware FP4->F16 convert, then one packed multiply by the block scale) and fed to
// v_mfma_f32_32x32x16_f16 with binary32 accumulation; the two tensor units are applied once to
// the accumulators.  The block scale byte b is placed in binary16 as (b & 0x7f) << 7, which is
// e4m3(b) * 2^-8 for normal and subnormal bytes alike; the 2^16 is folded into the unit product.
// The low-rank operands stay bf16 and use v_mfma_f32_32x32x16_bf16 on the same accumulators.
#include "metis_device.h"
#include "metis_host.h"

namespace metis {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int BK = 64;                 // K elements per main-loop step (4 scale blocks)
constexpr int LDS_PAD = 8;             // halves of padding per row: 144-byte row stride

// expand 8 packed codes (one dword) times the block scale (binary16 pair) into 8 halves
__device__ __forceinline__ uint4 expand8(uint32_t codes, half2_t sc)
{
    half2_t h0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 1.0f, 0) * sc;
    half2_t h1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 1.0f, 1) * sc;
    half2_t h2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 1.0f, 2) * sc;
    half2_t h3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 1.0f, 3) * sc;
    uint4 r;
    r.x = __builtin_bit_cast(uint32_t, h0);
    r.y = __builtin_bit_cast(uint32_t, h1);
    r.z = __builtin_bit_cast(uint32_t, h2);
    r.w = __builtin_bit_cast(uint32_t, h3);
    return r;
}
__device__ __forceinline__ half2_t scale_pair(uint32_t byte)
{
    const uint32_t h = (byte & 0x7fu) << 7;
    return __builtin_bit_cast(half2_t, h | (h << 16));
}

// Workgroup tile BM x BN, 256 threads = 4 waves in a 2 x 2 arrangement, each wave (BM/2) x (BN/2).
template <int BM, int BN, int OUT_F32>
__global__ __launch_bounds__(256) void gemm_nvfp4_kernel(
    const uint8_t* __restrict__ a_codes, const uint8_t* __restrict__ a_scales, const float* __restrict__ a_unit,
    const uint8_t* __restrict__ b_codes, const uint8_t* __restrict__ b_scales, const float* __restrict__ b_unit,
    int M, int N, int K, const uint16_t* __restrict__ t, const uint16_t* __restrict__ u, int r,
    const uint16_t* __restrict__ bias, void* __restrict__ out)
{
    constexpr int WM = BM / 2, WN = BN / 2;          // wave tile
    constexpr int TM = WM / 32, TN = WN / 32;        // 32x32 MFMA tiles per wave
    constexpr int STRIDE = BK + LDS_PAD;             // halves per LDS row
    __shared__ __attribute__((aligned(16))) uint16_t lds_a[BM * STRIDE];
    __shared__ __attribute__((aligned(16))) uint16_t lds_b[BN * STRIDE];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;

    float16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    const int kbytes = K / 2, kblocks = K / kBlock;
    // staging assignment: 16 bytes of codes (32 elements, 2 scale blocks) per thread-chunk
    constexpr int A_CHUNKS = BM * 2, B_CHUNKS = BN * 2;      // chunks per tile per K step (BK=64 -> 2 per row)

    for (int k0 = 0; k0 < K; k0 += BK) {
        // ---- global -> registers -> expand -> LDS
#pragma unroll
        for (int c = tid; c < A_CHUNKS + B_CHUNKS; c += 256) {
            const bool is_a = c < A_CHUNKS;
            const int cc = is_a ? c : c - A_CHUNKS;
            const int row = cc >> 1, half = cc & 1;
            const int grow = is_a ? min(m0 + row, M - 1) : min(n0 + row, N - 1);
            const int kk = k0 + half * 32;                    // first element of this chunk
            uint4 cw = make_uint4(0u, 0u, 0u, 0u);
            uint32_t sb = 0u;
            if (kk < K) {
                const uint8_t* cp = (is_a ? a_codes : b_codes) + (int64_t)grow * kbytes + kk / 2;
                const uint8_t* sp = (is_a ? a_scales : b_scales) + (int64_t)grow * kblocks + kk / kBlock;
                cw = *reinterpret_cast<const uint4*>(cp);     // K % 32 == 0: chunks never straddle the end
                sb = *reinterpret_cast<const uint16_t*>(sp);
            }
            const half2_t s0 = scale_pair(sb & 0xffu), s1 = scale_pair(sb >> 8);
            uint16_t* dst = (is_a ? lds_a : lds_b) + row * STRIDE + half * 32;
            reinterpret_cast<uint4*>(dst)[0] = expand8(cw.x, s0);
            reinterpret_cast<uint4*>(dst)[1] = expand8(cw.y, s0);
            reinterpret_cast<uint4*>(dst)[2] = expand8(cw.z, s1);
            reinterpret_cast<uint4*>(dst)[3] = expand8(cw.w, s1);
        }
        __syncthreads();
        // ---- MFMA over the staged step.  Operands are swapped (B fragment first) so that the four
        //      consecutive accumulator registers of a lane run along n, the contiguous output axis.
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            half8_t fa[TM], fb[TN];
            const int kofs = ks * 16 + (lane >> 5) * 8;
#pragma unroll
            for (int i = 0; i < TM; ++i)
                fa[i] = *reinterpret_cast<const half8_t*>(lds_a + (wm * WM + i * 32 + (lane & 31)) * STRIDE + kofs);
#pragma unroll
            for (int j = 0; j < TN; ++j)
                fb[j] = *reinterpret_cast<const half8_t*>(lds_b + (wn * WN + j * 32 + (lane & 31)) * STRIDE + kofs);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[j], fa[i], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // ---- tensor units (and the 2^8 * 2^8 of the scale placement)
    const float us = (*a_unit) * (*b_unit) * 65536.0f;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] *= us;

    // ---- bf16 low-rank extension: sum_j T[m,j] U[n,j], 32 columns per step
    for (int j0 = 0; j0 < r; j0 += 32) {
#pragma unroll
        for (int c = tid; c < (BM + BN) * 4; c += 256) {      // 16-byte chunks: 4 per row
            const bool is_a = c < BM * 4;
            const int cc = is_a ? c : c - BM * 4;
            const int row = cc >> 2, q = cc & 3;
            const int grow = is_a ? min(m0 + row, M - 1) : min(n0 + row, N - 1);
            const uint16_t* src = (is_a ? t : u) + (int64_t)grow * r + j0 + q * 8;
            uint16_t* dst = (is_a ? lds_a : lds_b) + row * STRIDE + q * 8;
            *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(src);
        }
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            bf16x8_t fa[TM], fb[TN];
            const int kofs = ks * 16 + (lane >> 5) * 8;
#pragma unroll
            for (int i = 0; i < TM; ++i)
                fa[i] = *reinterpret_cast<const bf16x8_t*>(lds_a + (wm * WM + i * 32 + (lane & 31)) * STRIDE + kofs);
#pragma unroll
            for (int j = 0; j < TN; ++j)
                fb[j] = *reinterpret_cast<const bf16x8_t*>(lds_b + (wn * WN + j * 32 + (lane & 31)) * STRIDE + kofs);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa[i], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // ---- epilogue.  acc[i][j][e]: n = 8*(e/4) + 4*(lane/32) + e%4, m = lane%32 within the tile
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = m0 + wm * WM + i * 32 + (lane & 31);
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = n0 + wn * WN + j * 32 + 8 * g + 4 * (lane >> 5);
                if (n >= N) continue;                          // N % 4 == 0 is required
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[e] = acc[i][j][4 * g + e];
                    if (bias) v[e] += bf16_lo(bias[n + e]);
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

int gemm_nvfp4(const void* a_codes, const void* a_scales, const float* a_unit, const void* b_codes, const void* b_scales,
               const float* b_unit, int64_t M, int64_t N, int64_t K, const void* t, const void* u, int64_t r,
               const void* bias, void* out, int out_dtype, hipStream_t st)
{
    if (!a_codes || !a_scales || !a_unit || !b_codes || !b_scales || !b_unit || !out) return METIS_E_ARG;
    if (M < 0 || N < 0 || K < 0 || r < 0) return METIS_E_ARG;
    if (out_dtype != METIS_DTYPE_BF16 && out_dtype != METIS_DTYPE_F32) return METIS_E_ARG;
    if (K % kBlock) return METIS_E_SHAPE;
    if (N % 4 || r % 32 || (r > 0 && (!t || !u))) return METIS_E_ARG;
    if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return METIS_E_ARG;
    if (((uintptr_t)a_codes % 16) || ((uintptr_t)b_codes % 16) || ((uintptr_t)a_scales % 2) || ((uintptr_t)b_scales % 2) ||
        ((uintptr_t)out % 16))
        return METIS_E_ARG;
    if (K % 32) return METIS_E_ARG;                            // 16-byte code chunks: rows must stay 16-byte aligned
    if (M == 0 || N == 0) return METIS_OK;
    constexpr int BM = 128, BN = 128;
    dim3 grid((unsigned)((N + BN - 1) / BN), (unsigned)((M + BM - 1) / BM));
    if (out_dtype == METIS_DTYPE_F32)
        hipLaunchKernelGGL((gemm_nvfp4_kernel<BM, BN, 1>), grid, dim3(256), 0, st, (const uint8_t*)a_codes,
                           (const uint8_t*)a_scales, a_unit, (const uint8_t*)b_codes, (const uint8_t*)b_scales, b_unit,
                           (int)M, (int)N, (int)K, (const uint16_t*)t, (const uint16_t*)u, (int)r, (const uint16_t*)bias, out);
    else
        hipLaunchKernelGGL((gemm_nvfp4_kernel<BM, BN, 0>), grid, dim3(256), 0, st, (const uint8_t*)a_codes,
                           (const uint8_t*)a_scales, a_unit, (const uint8_t*)b_codes, (const uint8_t*)b_scales, b_unit,
                           (int)M, (int)N, (int)K, (const uint16_t*)t, (const uint16_t*)u, (int)r, (const uint16_t*)bias, out);
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

}  // namespace metis
