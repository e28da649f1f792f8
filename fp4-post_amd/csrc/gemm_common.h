// Types and helpers shared by the GEMM translation units (metis_gemm.hip, metis_gemm_pipe.hip).
#pragma once
#include "metis_device.h"
#include "metis_host.h"

namespace metis {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
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
// bias[n]: bf16, or binary32 when bias_f32 is set (a bias that already carries a rank-one term, see nvfp4_gemv.hip)
__device__ __forceinline__ float bias_value(const uint16_t* bias, int bias_f32, int n)
{
    return bias_f32 ? reinterpret_cast<const float*>(bias)[n] : bf16_lo(bias[n]);
}
__device__ __forceinline__ half2_t scale_pair(uint32_t byte)
{
    const uint32_t h = (byte & 0x7fu) << 7;
    return __builtin_bit_cast(half2_t, h | (h << 16));
}

// Decode-sized GEMMs stream the packed weight rows straight from global memory into MFMA operands: lane l holds weight
// row n0 + l % 32, and per step the two half-waves cover 64 C consecutive elements of K, lane group l / 32 taking a
// contiguous run of 32 C elements (16 C bytes of codes, 2 C scale bytes).
template <int C>
struct RunRegs {
    uint4 c[C];                  // 32*C codes
    uint32_t sc[(C + 1) / 2];    // 2*C scale bytes
};

template <int C>
__device__ __forceinline__ void load_run(RunRegs<C>& r, const uint8_t* codes, const uint8_t* scales)
{
#pragma unroll
    for (int c = 0; c < C; ++c) r.c[c] = reinterpret_cast<const uint4*>(codes)[c];
    if constexpr (C == 1) r.sc[0] = *reinterpret_cast<const uint16_t*>(scales);
    else if constexpr (C == 2) r.sc[0] = *reinterpret_cast<const uint32_t*>(scales);
    else {
        const uint2 w = *reinterpret_cast<const uint2*>(scales);
        r.sc[0] = w.x; r.sc[1] = w.y;
    }
}

// The same with the distance between a run's 16-byte pieces as a run-time value: 16 for a row-major packed tensor, 1024
// for the decode layout of a weight (decode_weight_kernel: the pieces of the 64 lanes of a wave lie side by side, so one
// load instruction reads a KiB of consecutive bytes instead of 16 bytes from each of 64 rows).
template <int C>
__device__ __forceinline__ void load_run_strided(RunRegs<C>& r, const uint8_t* codes, int piece_stride, const uint8_t* scales)
{
#pragma unroll
    for (int c = 0; c < C; ++c) r.c[c] = *reinterpret_cast<const uint4*>(codes + (int64_t)c * piece_stride);
    if constexpr (C == 1) r.sc[0] = *reinterpret_cast<const uint16_t*>(scales);
    else if constexpr (C == 2) r.sc[0] = *reinterpret_cast<const uint32_t*>(scales);
    else {
        const uint2 w = *reinterpret_cast<const uint2*>(scales);
        r.sc[0] = w.x; r.sc[1] = w.y;
    }
}

// Decode layout of a packed weight [N, K], K % 256 == 0: for column tile T (rows 32 T .. 32 T + 31) and step `it`
// (256 elements of K) one block of kDecodeBlock bytes: four KiB of codes -- piece j of lane l = (h << 5 | row) at
// j * 1024 + l * 16 holds the row's code bytes [it * 128 + h * 64 + 16 j, + 16) -- then 512 bytes of scale bytes, lane l
// at 4096 + l * 8 holding the row's bytes [it * 16 + h * 8, + 8).  Rows past N are zero.  0.5625 B per element, as packed.

// MFMA operand m (8 elements) of a run
template <int C>
__device__ __forceinline__ half8_t run_operand(const RunRegs<C>& r, int m)
{
    const uint4 q = r.c[m >> 2];
    const uint32_t w = (m & 3) == 0 ? q.x : (m & 3) == 1 ? q.y : (m & 3) == 2 ? q.z : q.w;
    const uint32_t byte = (r.sc[m >> 3] >> (8 * ((m >> 1) & 3))) & 0xffu;
    return __builtin_bit_cast(half8_t, expand8(w, scale_pair(byte)));
}

// The same operand as the reference's bf16 arithmetic dequantizes it: bf16(bf16(e4m3 * unit) * e2m1), eight bf16 values
// (src/Metis/Metis/quant.py:33-36 evaluated in bf16, as under compute_dtype = bfloat16 in src/grpo/grpo.py:204-205).
template <int C>
__device__ __forceinline__ bf16x8_t run_operand_bf16(const RunRegs<C>& r, int m, float unit)
{
    typedef float float2_t __attribute__((ext_vector_type(2)));
    const uint4 q = r.c[m >> 2];
    const uint32_t w = (m & 3) == 0 ? q.x : (m & 3) == 1 ? q.y : (m & 3) == 2 ? q.z : q.w;
    const uint32_t byte = (r.sc[m >> 3] >> (8 * ((m >> 1) & 3))) & 0xffu;
    const float dq = rb(e4m3_value(byte) * unit);
    const float2_t p0 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 0);
    const float2_t p1 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 1);
    const float2_t p2 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 2);
    const float2_t p3 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 3);
    uint4 o;
    o.x = rb_pair(p0[0] * dq, p0[1] * dq);
    o.y = rb_pair(p1[0] * dq, p1[1] * dq);
    o.z = rb_pair(p2[0] * dq, p2[1] * dq);
    o.w = rb_pair(p3[0] * dq, p3[1] * dq);
    return __builtin_bit_cast(bf16x8_t, o);
}

// One weight matrix of a grouped decode-sized call, and the group: the column tiles (32 columns each) of the members are
// laid end to end.
constexpr int kMaxGroupMembers = 4;
struct SkinnyMember {
    const uint8_t* b_codes;
    const uint8_t* b_scales;
    const float* b_unit;
    const uint16_t* t;
    const uint16_t* u;
    const uint16_t* bias;
    void* out;
    float* part;                 // split-K partial sums of this member, nullptr when K is not split
    int N, r, tile_end, bias_f32, ldt;
    int decode;                  // b_codes is the weight in the decode layout (b_scales unused)
};
struct SkinnyGroup {
    SkinnyMember m[kMaxGroupMembers];
    int count, nsplit;
    const float* center;         // mean mode: binary32 [K], see skinny_tile
    int a_decode;                // the activation comes in the decode layout too (a_codes points at it, a_scales unused)
};

constexpr int L_BM = 256, L_BN = 256, L_STRIDE = BK + LDS_PAD;   // large-tile kernels: 256 x 256 per workgroup

// MFMA : VALU : LDS interleave requested from the scheduler for one K=16 sub-step of N_MFMA MFMAs
template <int N_MFMA, int N_VALU_PER_MFMA, int N_DSR, int N_DSW>
__device__ __forceinline__ void sched_substep()
{
#pragma unroll
    for (int m = 0; m < N_MFMA; ++m) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                       // one MFMA
        if (m < N_DSR) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);        // one LDS read
        if (N_VALU_PER_MFMA) __builtin_amdgcn_sched_group_barrier(0x002, N_VALU_PER_MFMA, 0);   // expansion VALU
        if (m < N_DSW) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);        // one LDS write
    }
}

// logical tile number -> origin of its 256 x 256 tile: groups of 4 tile-rows, walked column by column
__device__ __forceinline__ void tile_origin(int logical, int tiles_m, int tiles_n, int& m0, int& n0)
{
    constexpr int GM = 4;
    const int group = logical / (GM * tiles_n);
    const int first_m = group * GM;
    const int gsize = min(tiles_m - first_m, GM);
    const int tm = first_m + (logical % (GM * tiles_n)) % gsize;
    const int tn = (logical % (GM * tiles_n)) / gsize;
    m0 = tm * L_BM;
    n0 = tn * L_BN;
}

// Dynamic LDS above 64 KiB has to be allowed per kernel function and per device: done once for each pair.
inline int allow_dynamic_lds(const void* fn, size_t bytes, bool (&done)[64])
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return METIS_E_DEVICE;
    if (!done[dev]) {
        if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess) return METIS_E_DEVICE;
        done[dev] = true;
    }
    return METIS_OK;
}

// Sums the nsplit partial tiles of a split 256 x 256 GEMM (8 waves of 128 x 64) and writes the output.
// One wave per 32 x 64 piece (tile, wave of the GEMM, 32-row slab i): its lanes read what the same lanes of
// the GEMM wrote, 1 KiB per instruction, and add the splits in ascending order.
// The partial tiles hold the residual product only; the low-rank term t u^T (r > 0) is formed here, two 32 x 32 MFMA tiles
// per wave in ascending steps of 16 columns, and added with the bias.
// PB16 (every op of the reference rounded to bf16): the sum of the partial tiles is rounded to bf16 as the reference's
// bf16 matmul rounds it, the bias is added in bf16, then the low-rank term and the final rounding.
template <int OUT_F32, int PB16 = 0>
__global__ __launch_bounds__(64) void gemm_splitk_reduce_kernel(const float* __restrict__ ws, int nsplit, int M, int N,
                                                                int tiles_m, int tiles_n, void* __restrict__ out, int nfull,
                                                                const uint16_t* __restrict__ bias, int bias_f32,
                                                                const uint16_t* __restrict__ t = nullptr,
                                                                const uint16_t* __restrict__ u = nullptr, int r = 0)
{
    constexpr int TN = 2, WTN = 64, NTHREADS = 512, TILE = L_BM * L_BN;
    __shared__ __attribute__((aligned(16))) uint16_t cw[32 * 72];
    const int total = tiles_m * tiles_n - nfull;                 // split tiles
    const int tile = blockIdx.x >> 5, wave = (blockIdx.x >> 2) & 7, i = blockIdx.x & 3;
    const int lane = threadIdx.x, tid = wave * 64 + lane;
    const int wm = wave / 4, wn = wave % 4;
    int m0, n0;
    tile_origin(nfull + tile, tiles_m, tiles_n, m0, n0);
    const int mbase = m0 + wm * 128 + i * 32, nbase = n0 + wn * WTN;
    if (mbase >= M || nbase >= N) return;

    float4 v[TN][4];
    const float* src = ws + (size_t)tile * TILE + (size_t)(i * TN * 4) * (NTHREADS * 4) + tid * 4;
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) v[j][g] = *reinterpret_cast<const float4*>(src + (j * 4 + g) * (NTHREADS * 4));
    for (int z = 1; z < nsplit; ++z) {
        const float* sz = src + (size_t)z * total * TILE;
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const float4 p = *reinterpret_cast<const float4*>(sz + (j * 4 + g) * (NTHREADS * 4));
                v[j][g].x += p.x; v[j][g].y += p.y; v[j][g].z += p.z; v[j][g].w += p.w;
            }
    }
    float16_t low[TN];                                           // the low-rank term t u^T of this piece
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) low[j][e] = 0.0f;
    {
        if (r > 0) {                                             // lane l: row l % 32 of its operand, columns 8 (l / 32) .. of the step
            const uint16_t* tp = t + (int64_t)min(mbase + (lane & 31), M - 1) * r + 8 * (lane >> 5);
            const uint16_t* up[TN];
#pragma unroll
            for (int j = 0; j < TN; ++j) up[j] = u + (int64_t)min(nbase + j * 32 + (lane & 31), N - 1) * r + 8 * (lane >> 5);
            for (int k0 = 0; k0 < r; k0 += 16) {
                const bf16x8_t ga = *reinterpret_cast<const bf16x8_t*>(tp + k0);
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    low[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const bf16x8_t*>(up[j] + k0), ga, low[j], 0, 0, 0);
            }
        }
    }
    if constexpr (PB16 == 0) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = nbase + j * 32 + 8 * g + 4 * (lane >> 5);
                float q[4] = {v[j][g].x, v[j][g].y, v[j][g].z, v[j][g].w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    q[e] += low[j][4 * g + e];
                    if (bias) q[e] += bias_value(bias, bias_f32, min(n + e, N - 1));
                }
                v[j][g] = make_float4(q[0], q[1], q[2], q[3]);
            }
    } else {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = nbase + j * 32 + 8 * g + 4 * (lane >> 5);
                float q[4] = {rb(v[j][g].x), rb(v[j][g].y), rb(v[j][g].z), rb(v[j][g].w)};
                if (bias) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) q[e] = rb(q[e] + bias_value(bias, bias_f32, min(n + e, N - 1)));
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) q[e] += low[j][4 * g + e];
                v[j][g] = make_float4(rb(q[0]), rb(q[1]), rb(q[2]), rb(q[3]));
            }
    }

    if (!OUT_F32 && (N & 7) == 0) {
        // 32 x 64 bf16 through LDS: a store instruction then writes 8 rows x 128 contiguous bytes
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                uint2 w;
                w.x = bf16_bits(v[j][g].x) | (bf16_bits(v[j][g].y) << 16);
                w.y = bf16_bits(v[j][g].z) | (bf16_bits(v[j][g].w) << 16);
                *reinterpret_cast<uint2*>(cw + (lane & 31) * 72 + j * 32 + 8 * g + 4 * (lane >> 5)) = w;
            }
        __syncthreads();
        const int rsub = lane >> 3, chunk = lane & 7;
        const int n = nbase + chunk * 8;
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int ml = it * 8 + rsub;
            const uint4 w = *reinterpret_cast<const uint4*>(cw + ml * 72 + chunk * 8);
            if (mbase + ml < M && n < N) *reinterpret_cast<uint4*>((uint16_t*)out + (int64_t)(mbase + ml) * N + n) = w;
        }
        return;
    }
    const int m = mbase + (lane & 31);
    if (m >= M) return;
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int n = nbase + j * 32 + 8 * g + 4 * (lane >> 5);
            if (n >= N) continue;                                  // N % 4 == 0
            if (OUT_F32) {
                *reinterpret_cast<float4*>((float*)out + (int64_t)m * N + n) = v[j][g];
            } else {
                uint2 w;
                w.x = bf16_bits(v[j][g].x) | (bf16_bits(v[j][g].y) << 16);
                w.y = bf16_bits(v[j][g].z) | (bf16_bits(v[j][g].w) << 16);
                *reinterpret_cast<uint2*>((uint16_t*)out + (int64_t)m * N + n) = w;
            }
        }
}

// Splits of K for a tiled GEMM.  A shape that would leave more than half of the compute units without a tile is
// split whole: as many workgroups per tile as fill the device once, at least 8 K steps (512 elements) each, at
// most 16.  A shape whose last round of tiles covers at most half of the units has only those tiles split; the
// full rounds before it run unsplit (up to four of them: measured gains 6-28 % at 1-4 full rounds, a loss of 2 % at
// nine, where the rounds have drifted apart enough to hide the tail anyway).  nsplit = 1: do not split.
struct SplitPlan {
    int nsplit;
    int nfull;                   // leading tiles that run unsplit (a multiple of the compute units)
};
inline SplitPlan split_plan(int64_t M, int64_t N, int64_t K)
{
    const SplitPlan none = {1, 0};
    if (M < L_BM || N < L_BN || K % BK) return none;
    const int64_t tiles = ((M + L_BM - 1) / L_BM) * ((N + L_BN - 1) / L_BN);
    const int cus = device_cus();
    if (cus <= 0 || cus % 8 || tiles > INT32_MAX) return none;
    int64_t part = tiles, nfull = 0;                            // tiles to split
    if (tiles * 2 > cus) {
        part = tiles % cus;
        nfull = tiles - part;
        if (tiles < cus || part == 0 || part * 2 > cus || nfull > 4 * (int64_t)cus || false) return none;
    }
    int64_t s = cus / part;
    if (s > K / BK / 8) s = K / BK / 8;
    if (s > 16) s = 16;
    if (s < 2) return none;
    return SplitPlan{(int)s, (int)nfull};
}

}  // namespace metis
