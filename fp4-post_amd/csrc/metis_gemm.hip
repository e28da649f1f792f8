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
#include "gemm_common.h"
#include "nvfp4_encode.h"
#include "lowrank_small_steps.h"
#include <stdlib.h>
#include <type_traits>

namespace metis {

// (measure_env(), metis_host.h: kernel variants and shape overrides of a -DMETIS_MEASURE build)

// Workgroup tile BM x BN, 256 threads = 4 waves in a 2 x 2 arrangement, each wave (BM/2) x (BN/2).
template <int BM, int BN, int OUT_F32>
__global__ __launch_bounds__(256) void gemm_nvfp4_kernel(
    const uint8_t* __restrict__ a_codes, const uint8_t* __restrict__ a_scales, const float* __restrict__ a_unit,
    const uint8_t* __restrict__ b_codes, const uint8_t* __restrict__ b_scales, const float* __restrict__ b_unit,
    int M, int N, int K, const uint16_t* __restrict__ t, const uint16_t* __restrict__ u, int r,
    const uint16_t* __restrict__ bias, void* __restrict__ out, int bias_f32)
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

// ---------------------------------------------------------------------------------------------
// Large-tile kernel: 256 x 256 per workgroup, K step 64, LDS double buffered (2 x 72 KiB) with one
// barrier per step.  Two wave layouts:
//   4 waves (2 x 2), 128 x 128 per wave: 16 MFMA tiles, 256 accumulator registers per lane
//   8 waves (2 x 4), 128 x  64 per wave:  8 MFMA tiles, two waves per SIMD
// Each thread owns one (8 waves) or two (4 waves) rows of the 512-row A|B tile per step: it fetches
// their 32 bytes of codes and 4 scale bytes into registers a full step ahead and expands them into
// the idle LDS buffer between the MFMAs of the current buffer.
//
// Tile order: workgroup ids are dealt round-robin to the 8 XCDs by the hardware, so id -> (xcd,
// slot) is undone first to give every XCD (and its private L2) one contiguous range of tiles,
// which is then walked in groups of 4 tile-rows so that concurrently running workgroups share
// A and B panels.
// ---------------------------------------------------------------------------------------------
constexpr int L_STAGE_HALVES = (L_BM + L_BN) * L_STRIDE;          // one buffer: A rows then B rows

struct RowRegs {
    uint4 c0, c1;      // 64 codes
    uint32_t sc;       // 4 scale bytes
};

__device__ __forceinline__ void expand_row(const RowRegs& r, uint16_t* dst)
{
    const half2_t s0 = scale_pair(r.sc & 0xffu), s1 = scale_pair((r.sc >> 8) & 0xffu);
    const half2_t s2 = scale_pair((r.sc >> 16) & 0xffu), s3 = scale_pair(r.sc >> 24);
    uint4* d = reinterpret_cast<uint4*>(dst);
    d[0] = expand8(r.c0.x, s0); d[1] = expand8(r.c0.y, s0);
    d[2] = expand8(r.c0.z, s1); d[3] = expand8(r.c0.w, s1);
    d[4] = expand8(r.c1.x, s2); d[5] = expand8(r.c1.y, s2);
    d[6] = expand8(r.c1.z, s3); d[7] = expand8(r.c1.w, s3);
}

// one expand8 (8 elements) of a row: p in 0..7
template <bool STORE = true>
__device__ __forceinline__ void expand_piece(const RowRegs& r, int p, uint16_t* d)
{
    const uint32_t w = p == 0 ? r.c0.x : p == 1 ? r.c0.y : p == 2 ? r.c0.z : p == 3 ? r.c0.w
                     : p == 4 ? r.c1.x : p == 5 ? r.c1.y : p == 6 ? r.c1.z : r.c1.w;
    const uint4 e = expand8(w, scale_pair((r.sc >> (8 * (p >> 1))) & 0xffu));
    if (STORE) reinterpret_cast<uint4*>(d)[p] = e;
    else asm volatile("" ::"v"(e.x), "v"(e.y), "v"(e.z), "v"(e.w));      // measurement: the arithmetic without the LDS write
}

// SPLIT: tiles nfull .. total-1 have nsplit workgroups each, every one contracting its own range of K steps and
// leaving its binary32 tile (units applied; low-rank term and bias in split 0 only) in
// ws[split * (total - nfull) + tile - nfull][65536], ordered as the accumulator registers lie, for
// gemm_splitk_reduce_kernel.  nfull = 0 splits every tile (shapes with few tiles); nfull > 0 splits only the
// last, partial round of a shape whose tile count is a little over a multiple of the compute units.
template <int OUT_F32, int WN_WAVES, int DBG = 0, int SPLIT = 0>
__global__ __launch_bounds__(128 * WN_WAVES, 1) void gemm_nvfp4_large_kernel(
    const uint8_t* __restrict__ a_codes, const uint8_t* __restrict__ a_scales, const float* __restrict__ a_unit,
    const uint8_t* __restrict__ b_codes, const uint8_t* __restrict__ b_scales, const float* __restrict__ b_unit,
    int M, int N, int K, const uint16_t* __restrict__ t, const uint16_t* __restrict__ u, int r,
    const uint16_t* __restrict__ bias, void* __restrict__ out, int tiles_m, int tiles_n, float* __restrict__ ws,
    int nsplit, int bias_f32, int nfull)
{
    extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
    constexpr int TM = 4;                            // 32-tall MFMA tiles per wave along m
    constexpr int TN = 8 / WN_WAVES;                 // 32-wide MFMA tiles per wave along n: 4 or 2
    constexpr int WTN = 256 / WN_WAVES;              // wave tile width: 128 or 64
    constexpr int NTHREADS = 128 * WN_WAVES;
    constexpr int RPT = 512 / NTHREADS;              // A|B tile rows expanded by one thread: 2 or 1
    constexpr int PIECES = 8 * RPT;                  // expand8 pieces per thread per step
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN_WAVES, wn = wave % WN_WAVES;

    // ---- tile assignment (XCD-contiguous, grouped).  SPLIT: the first nfull tiles (a multiple of 8) run unsplit,
    //      every XCD its share of them first; the remaining tiles have nsplit workgroups each.
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
    const int steps_all = K / BK;
    const int step_begin = partial ? (int)((int64_t)split * steps_all / nsplit) : 0;
    const int step_end = partial ? (int)((int64_t)(split + 1) * steps_all / nsplit) : steps_all;

    float16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    // ---- rows of the A|B tile this thread stages: tile row q*NTHREADS + tid (0..255 = A, 256..511 = B)
    const int kbytes = K / 2, kblocks = K / kBlock;
    const uint8_t* cp[RPT];
    const uint8_t* sp[RPT];
    int lds_row[RPT];
#pragma unroll
    for (int q = 0; q < RPT; ++q) {
        const int trow = q * NTHREADS + tid;
        const bool is_a = trow < L_BM;
        const int64_t grow = is_a ? min(m0 + trow, M - 1) : min(n0 + trow - L_BM, N - 1);
        cp[q] = (is_a ? a_codes : b_codes) + grow * kbytes + step_begin * (BK / 2);
        sp[q] = (is_a ? a_scales : b_scales) + grow * kblocks + step_begin * (BK / kBlock);
        lds_row[q] = trow * L_STRIDE;
    }
    auto fetch = [&](RowRegs (&rr)[RPT], int k0) {               // K % 64 == 0: always a full step
#pragma unroll
        for (int q = 0; q < RPT; ++q) {
            rr[q].c0 = reinterpret_cast<const uint4*>(cp[q] + k0 / 2)[0];
            rr[q].c1 = reinterpret_cast<const uint4*>(cp[q] + k0 / 2)[1];
            rr[q].sc = *reinterpret_cast<const uint32_t*>(sp[q] + k0 / kBlock);
        }
    };

    const int steps = step_end - step_begin;                     // >= 1: the host never asks for more splits than steps
    // r1: rows of step s+1, expanded during step s; r2: rows of step s+2, in flight during step s
    RowRegs r1[RPT], r2[RPT];
    fetch(r1, 0);
#pragma unroll
    for (int q = 0; q < RPT; ++q) expand_row(r1[q], lds + lds_row[q]);
    if (steps > 1) fetch(r1, BK);
    __syncthreads();

    const int frag_off = (lane & 31) * L_STRIDE + (lane >> 5) * 8;
    const int a_off = wm * 128 * L_STRIDE + frag_off;
    const int b_off = (L_BM + wn * WTN) * L_STRIDE + frag_off;
    half8_t fa[2][TM], fb[2][TN];
    auto load_frags = [&](int buf, const uint16_t* stage, int ks) {
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[buf][i] = *reinterpret_cast<const half8_t*>(stage + a_off + i * 32 * L_STRIDE + ks * 16);
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[buf][j] = *reinterpret_cast<const half8_t*>(stage + b_off + j * 32 * L_STRIDE + ks * 16);
    };
    auto mfmas = [&](int buf) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[buf][j], fa[buf][i], acc[i][j], 0, 0, 0);
    };
    constexpr int NM = TM * TN, NF = TM + TN;
    // pieces expanded in sub-steps 0, 1, 2 (all before the barrier)
    constexpr int P0 = (PIECES + 2) / 3, P1 = (PIECES - P0 + 1) / 2, P2 = PIECES - P0 - P1;
    constexpr int VPM = (P0 * 9 + NM - 1) / NM;       // VALU ops to slot behind each MFMA
    // One K step.  EXPAND: rows of step s+1 (r1) are expanded into the idle LDS buffer during sub-steps
    // 0..2; the barrier sits before sub-step 3, whose MFMAs cover the first fragment loads of step s+1.
    // FETCH: global loads of step s+2 into r2, issued at the top so they have the whole step to arrive.
    auto stage = [&](int s, auto do_expand, auto do_fetch) {
        constexpr bool EXPAND = decltype(do_expand)::value && !(DBG & 1), FETCH = decltype(do_fetch)::value && !(DBG & 1);
        const uint16_t* cur = lds + (s & 1) * L_STAGE_HALVES;
        uint16_t* nxt = lds + ((s + 1) & 1) * L_STAGE_HALVES;
        if (FETCH) fetch(r2, (s + 2) * BK);
        auto pieces = [&](int from, int to) {
#pragma unroll
            for (int p = from; p < to; ++p) expand_piece<!(DBG & 4)>(r1[p / 8], p % 8, nxt + lds_row[p / 8]);
        };
        load_frags(1, cur, 1);
        if (EXPAND) pieces(0, P0);
        mfmas(0);
        if (EXPAND) sched_substep<NM, VPM, NF, P0>(); else sched_substep<NM, 0, NF, 0>();
        load_frags(0, cur, 2);
        if (EXPAND) pieces(P0, P0 + P1);
        mfmas(1);
        if (EXPAND) sched_substep<NM, VPM, NF, P1>(); else sched_substep<NM, 0, NF, 0>();
        load_frags(1, cur, 3);
        if (EXPAND) pieces(P0 + P1, PIECES);
        mfmas(0);
        if (EXPAND) sched_substep<NM, VPM, NF, P2>(); else sched_substep<NM, 0, NF, 0>();
        if (!(DBG & 2)) __syncthreads();
        if (EXPAND || (DBG & 1)) load_frags(0, nxt, 0);
        mfmas(1);
        sched_substep<NM, 0, NF, 0>();
        if (FETCH) {
#pragma unroll
            for (int q = 0; q < RPT; ++q) r1[q] = r2[q];
        }
    };
    using T_ = std::true_type;
    using F_ = std::false_type;
    load_frags(0, lds, 0);
    int s = 0;
    for (; s + 2 < steps; ++s) stage(s, T_{}, T_{});
    if (s + 1 < steps) { stage(s, T_{}, F_{}); ++s; }
    stage(s, F_{}, F_{});
    __syncthreads();

    // ---- tensor units (and the 2^8 * 2^8 of the scale placement)
    const float us = (*a_unit) * (*b_unit) * 65536.0f;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] *= us;

    if (SPLIT && split) {                                        // the low-rank term and the bias enter once
        r = 0;
        bias = nullptr;
    }
    // ---- bf16 low-rank extension, 32 columns of T / U per step, staged in buffer 0
    for (int j0 = 0; j0 < r; j0 += 32) {
#pragma unroll
        for (int q = 0; q < RPT; ++q) {
            const int trow = q * NTHREADS + tid;
            const bool is_a = trow < L_BM;
            const int64_t grow = is_a ? min(m0 + trow, M - 1) : min(n0 + trow - L_BM, N - 1);
            const uint4* src = reinterpret_cast<const uint4*>((is_a ? t : u) + grow * r + j0);
            uint4* dst = reinterpret_cast<uint4*>(lds + lds_row[q]);
#pragma unroll
            for (int c = 0; c < 4; ++c) dst[c] = src[c];
        }
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            bf16x8_t ga[TM], gb[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) ga[i] = *reinterpret_cast<const bf16x8_t*>(lds + a_off + i * 32 * L_STRIDE + ks * 16);
#pragma unroll
            for (int j = 0; j < TN; ++j) gb[j] = *reinterpret_cast<const bf16x8_t*>(lds + b_off + j * 32 * L_STRIDE + ks * 16);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gb[j], ga[i], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    if (SPLIT != 0 && partial) {
        float* wt = ws + (size_t)(split * (total - nfull) + (logical - nfull)) * (L_BM * L_BN) + tid * 4;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int n = n0 + wn * WTN + j * 32 + 8 * g + 4 * (lane >> 5);
                    float v[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        v[e] = acc[i][j][4 * g + e];
                        if (bias) v[e] += bias_value(bias, bias_f32, min(n + e, N - 1));
                    }
                    *reinterpret_cast<float4*>(wt + ((i * TN + j) * 4 + g) * (NTHREADS * 4)) = make_float4(v[0], v[1], v[2], v[3]);
                }
        return;
    }
    // ---- epilogue, bf16 output with N % 8 == 0: each wave transposes its tile through its own slice of the
    //      (now idle) LDS so that a store instruction writes 8 rows x 128 contiguous bytes instead of 32 rows x 16
    if constexpr (!OUT_F32 && WN_WAVES == 4) {
        if ((N & 7) == 0) {
            constexpr int CROW = 64 + 8;                              // halves per staged row (144 bytes: conflict-free)
            uint16_t* cw = lds + wave * (128 * CROW);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int nl = j * 32 + 8 * g + 4 * (lane >> 5);
                        float v[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            v[e] = acc[i][j][4 * g + e];
                            if (bias) v[e] += bias_value(bias, bias_f32, min(n0 + wn * WTN + nl + e, N - 1));
                        }
                        uint2 w;
                        w.x = bf16_bits(v[0]) | (bf16_bits(v[1]) << 16);
                        w.y = bf16_bits(v[2]) | (bf16_bits(v[3]) << 16);
                        *reinterpret_cast<uint2*>(cw + (i * 32 + (lane & 31)) * CROW + nl) = w;
                    }
            // same wave reads back what it wrote: no workgroup barrier needed, only the wave's own LDS writes
            __builtin_amdgcn_s_waitcnt(0xC07F);                       // lgkmcnt(0)
            const int rsub = lane >> 3, chunk = lane & 7;
            const int n = n0 + wn * WTN + chunk * 8;
#pragma unroll
            for (int it = 0; it < 16; ++it) {
                const int ml = it * 8 + rsub;
                const int m = m0 + wm * 128 + ml;
                const uint4 w = *reinterpret_cast<const uint4*>(cw + ml * CROW + chunk * 8);
                if (m < M && n < N) *reinterpret_cast<uint4*>((uint16_t*)out + (int64_t)m * N + n) = w;
            }
            return;
        }
    }
    // ---- epilogue.  acc[i][j][e]: n = 8*(e/4) + 4*(lane/32) + e%4, m = lane%32 within the tile
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = m0 + wm * 128 + i * 32 + (lane & 31);
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = n0 + wn * WTN + j * 32 + 8 * g + 4 * (lane >> 5);
                if (n >= N) continue;
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

size_t gemm_grouped_workspace_bytes(int64_t M, int64_t K, const GemmMember* members, int count);

size_t gemm_workspace_bytes(int64_t M, int64_t N, int64_t K)
{
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    if (M < 256) {                                            // skinny kernel
        const GemmMember g = {nullptr, nullptr, nullptr, nullptr, nullptr, 0, nullptr, nullptr, N, 0, 0};
        return gemm_grouped_workspace_bytes(M, K, &g, 1);
    }
    const SplitPlan p = split_plan(M, N, K);
    if (p.nsplit <= 1) return 0;
    const int64_t tiles = ((M + L_BM - 1) / L_BM) * ((N + L_BN - 1) / L_BN);
    return (size_t)p.nsplit * (size_t)(tiles - p.nfull) * L_BM * L_BN * sizeof(float);
}

template <int WN_WAVES>
static int launch_large(const void* a_codes, const void* a_scales, const float* a_unit, const void* b_codes,
                        const void* b_scales, const float* b_unit, int64_t M, int64_t N, int64_t K, const void* t,
                        const void* u, int64_t r, const void* bias, void* out, int out_dtype, hipStream_t st,
                        int bias_f32 = 0, float* ws = nullptr, int nsplit = 1, int nfull = 0)
{
    static bool attr_set[4][64] = {};
    const size_t lds_bytes = 2 * (size_t)L_STAGE_HALVES * sizeof(uint16_t);
    const bool split = WN_WAVES == 4 && ws && nsplit > 1;
    const int f32 = out_dtype == METIS_DTYPE_F32;
    const void* fn = split ? (f32 ? (const void*)gemm_nvfp4_large_kernel<1, WN_WAVES, 0, WN_WAVES == 4>
                                  : (const void*)gemm_nvfp4_large_kernel<0, WN_WAVES, 0, WN_WAVES == 4>)
                   : f32   ? (const void*)gemm_nvfp4_large_kernel<1, WN_WAVES>
                           : (const void*)gemm_nvfp4_large_kernel<0, WN_WAVES>;
#ifdef METIS_MEASURE
    const char* d = getenv("METIS_GEMM_DBG");                  // results are meaningless:
    const int v = d ? atoi(d) : 0;                             // 1 = no operand fetch/expansion, 7 = also no barriers,
                                                               // 4 = expansion arithmetic without its LDS writes
    if (v == 1 || v == 7 || v == 4) {
        fn = v == 1 ? (const void*)gemm_nvfp4_large_kernel<0, WN_WAVES, 1> : v == 4 ? (const void*)gemm_nvfp4_large_kernel<0, WN_WAVES, 4> : (const void*)gemm_nvfp4_large_kernel<0, WN_WAVES, 7>;
        if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes) != hipSuccess) return METIS_E_DEVICE;
    } else
#endif
    if (const int rc = allow_dynamic_lds(fn, lds_bytes, attr_set[(split ? 2 : 0) + f32])) {
        return rc;
    }
    const int tiles_m = (int)((M + L_BM - 1) / L_BM), tiles_n = (int)((N + L_BN - 1) / L_BN);
    const int total = tiles_m * tiles_n;
    if (!split) { nsplit = 1; nfull = 0; }
    // per XCD: its share of the unsplit tiles, then its share of the split ones
    const unsigned grid_x = split ? 8u * (unsigned)(nfull / 8 + ((total - nfull) * nsplit + 7) / 8)
                                  : (unsigned)(((total + 7) / 8) * 8);
    const uint8_t *ac = (const uint8_t*)a_codes, *as = (const uint8_t*)a_scales, *bc = (const uint8_t*)b_codes,
                  *bs = (const uint8_t*)b_scales;
    const uint16_t *tp = (const uint16_t*)t, *up = (const uint16_t*)u, *bp = (const uint16_t*)bias;
    int Mi = (int)M, Ni = (int)N, Ki = (int)K, ri = (int)r, tmi = tiles_m, tni = tiles_n;
    void* args[] = {&ac, &as, &a_unit, &bc, &bs, &b_unit, &Mi, &Ni, &Ki, &tp, &up, &ri, &bp, &out, &tmi, &tni, &ws, &nsplit, &bias_f32, &nfull};
    if (hipLaunchKernel(fn, dim3(grid_x), dim3(128 * WN_WAVES), args, lds_bytes, st) != hipSuccess) {
        (void)hipGetLastError();
        return METIS_E_LAUNCH;
    }
    if (split) {
        const dim3 rgrid((unsigned)(total - nfull) * 32u);
        if (f32)
            hipLaunchKernelGGL((gemm_splitk_reduce_kernel<1, 0>), rgrid, dim3(64), 0, st, ws, nsplit, Mi, Ni, tmi, tni, out, nfull, (const uint16_t*)nullptr, 0);
        else
            hipLaunchKernelGGL((gemm_splitk_reduce_kernel<0, 0>), rgrid, dim3(64), 0, st, ws, nsplit, Mi, Ni, tmi, tni, out, nfull, (const uint16_t*)nullptr, 0);
        if (hipGetLastError() != hipSuccess) return METIS_E_LAUNCH;
    }
    return METIS_OK;
}

// ---------------------------------------------------------------------------------------------
// Skinny kernel for M <= 64 per workgroup row (decode steps, small batches): HBM-bound on the packed
// weight bytes; taller inputs below 256 rows take one grid row per 64 rows.
// No LDS in the main loop and no barriers: a workgroup owns 32 output columns, its eight waves
// split K between them, and every wave streams its slice of the 32 weight rows straight from
// global memory into MFMA operands (the activations, at most 64 rows, come from L2).
//
// Lane l holds weight row n0 + l % 32; per iteration the two half-waves cover 64*C consecutive
// elements of K, lane group l / 32 taking a contiguous run of 32*C elements (16*C bytes of codes,
// 2*C scale bytes), so that with C = 4 the two lanes of a row consume one whole 128-byte line.
// A contraction may visit K in any order as long as both operands agree: the m-th MFMA of an
// iteration multiplies elements [8m, 8m+8) of every lane's run, and the activation rows are
// fetched with the same mapping.  Partial sums of the eight waves meet in LDS at the end.
// ---------------------------------------------------------------------------------------------
// CEN: the activation is a centred residual, X^ = 1 me^T + R (mean mode).  The workgroup's slice of the binary32
// centre me is staged in LDS (in the reduction buffer, idle during the main loop) as binary16 pairs hi + lo
// (22 significant bits, prescaled by 2^-4: |me| < 2^20) and enters as one more MFMA per step against the weight
// operand that has just been expanded: a pseudo activation tile whose even rows are hi and odd rows lo.  The packed
// weight is read once for R W^T and for the rank-one term 1 (W^ me)^T, at the cost of half as many MFMAs again
// on a kernel that is bound elsewhere.
//
// PB16: the layer's arithmetic is bf16 and the forward follows the reference's all-bf16 evaluation
// (src/Metis/Metis/bitlinear.py:435-438 under compute_dtype = bfloat16, src/grpo/grpo.py:204-205): both operands are its
// twice-rounded bf16 dequantized values (bf16 MFMA, no unit factor), the residual product is rounded to bf16 as its
// bf16 matmul rounds it, the bias is added in bf16, then the low-rank term and one final rounding.  The low-rank
// products therefore stay apart from the residual sums: they pass through the reduction buffer a second time (K slice 0
// leaves them as one more partial in slot nsplit when K is split).
//
// ADENSE = 2: the packed activation comes in the decode layout, like a cached weight.
// ADENSE = 1: the activation arrives as ready 16-bit MFMA operands (skinny_operand_kernel: one 16-byte piece per lane and
// MFMA, a coalesced KiB per load instruction) instead of packed codes that every workgroup would expand again: the
// vector unit is left with the weight operand alone.  a_codes then points at that buffer and a_scales is unused.
template <int TM, int C, int WAVES, int OUT_F32, int CEN = 0, int PB16 = 0, int ADENSE = 0>
__device__ __forceinline__ void skinny_tile(
    const uint8_t* __restrict__ a_codes, const uint8_t* __restrict__ a_scales, const float* __restrict__ a_unit,
    const uint8_t* __restrict__ b_codes, const uint8_t* __restrict__ b_scales, const float* __restrict__ b_unit,
    int M, int N, int K, const uint16_t* __restrict__ t, const uint16_t* __restrict__ u, int r,
    const uint16_t* __restrict__ bias, void* __restrict__ out, int bias_f32, int n0, int ldt,
    float* __restrict__ part, int nsplit, const float* __restrict__ center = nullptr, int decode = 0)
{
    __shared__ __attribute__((aligned(16))) float red[WAVES][TM * 16][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, hi = lane >> 5;
    const int m0 = blockIdx.y * 32 * TM;
    const int kbytes = K / 2, kblocks = K / kBlock;
    const int nrow = min(n0 + (lane & 31), N - 1);
    // the weight: row-major packed (a lane walks its row), or the decode layout (a wave walks the blocks of its column tile)
    const uint8_t* bc = b_codes + (int64_t)nrow * kbytes + hi * 16 * C;
    const uint8_t* bs = b_scales + (int64_t)nrow * kblocks + hi * 2 * C;
    int w_step = 32 * C, w_piece = 16, ws_step = 4 * C;
    if (C == 4 && decode) {
        const uint8_t* tile0 = b_codes + (int64_t)(n0 / 32) * (K / 256) * kDecodeBlock;
        bc = tile0 + lane * 16;
        bs = tile0 + 4096 + lane * 8;
        w_step = kDecodeBlock; w_piece = 1024; ws_step = kDecodeBlock;
    }
    static_assert(ADENSE != 1 || CEN == 0, "ready operands carry no centre");
    static_assert(ADENSE == 0 || C == 4, "ready operands and the decode layout come in the wide-run layout");
    const uint8_t *ac[TM], *as[TM];
    const uint4* ap[TM];
    // the activation likewise: row-major packed (64 lanes read 64 different lines per load instruction), or its decode
    // layout (one KiB of consecutive bytes per load instruction; rows past M are zero there)
    constexpr bool a_dec = ADENSE == 2;
    constexpr int a_step = a_dec ? kDecodeBlock : 32 * C, a_piece = a_dec ? 1024 : 16, as_step = a_dec ? kDecodeBlock : 4 * C;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int mrow = min(m0 + i * 32 + (lane & 31), M - 1);
        ac[i] = a_codes + (int64_t)mrow * kbytes + hi * 16 * C;
        as[i] = a_scales + (int64_t)mrow * kblocks + hi * 2 * C;
        if constexpr (a_dec) {
            const uint8_t* tile0 = a_codes + (int64_t)(m0 / 32 + i) * (K / 256) * kDecodeBlock;
            ac[i] = tile0 + lane * 16;
            as[i] = tile0 + 4096 + lane * 8;
        }
        // operand (row tile, iteration, m): 64 lanes x 16 bytes
        ap[i] = reinterpret_cast<const uint4*>(a_codes) + (int64_t)(m0 / 32 + i) * (K / (64 * C)) * (4 * C * 64) + lane;
    }
    float16_t acc[TM];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][e] = 0.0f;

    // K slice of this workgroup (grid z; the whole of K when part == nullptr), dealt to the waves
    const int iters_all = K / (64 * C);
    const int slice = part ? (int)blockIdx.z : 0;
    const int s0 = part ? slice * iters_all / nsplit : 0;
    const int iters = (part ? (slice + 1) * iters_all / nsplit : iters_all) - s0;
    const int it1 = s0 + (wave + 1) * iters / WAVES;
    float* mes = &red[0][0][0];
    float16_t accm;                                            // CEN: the pseudo tile (even lanes: B . hi, odd lanes: B . lo)
#pragma unroll
    for (int e = 0; e < 16; ++e) accm[e] = 0.0f;
    if constexpr (CEN != 0) {                                  // the host has checked that the slice fits
        // 32 bytes per 8 elements: [hi x 8 | lo x 8]
        const int klen = iters * 64 * C;
        const float* src = center + (int64_t)s0 * 64 * C;
        for (int k = threadIdx.x * 4; k < klen; k += 64 * WAVES * 4) {
            const float4 f = *reinterpret_cast<const float4*>(src + k);
            const float v[4] = {f.x * 0.0625f, f.y * 0.0625f, f.z * 0.0625f, f.w * 0.0625f};
            half4_t h, l;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                h[j] = (_Float16)v[j];
                l[j] = (_Float16)(v[j] - (float)h[j]);
            }
            char* d = reinterpret_cast<char*>(mes) + (k >> 3) * 32 + ((k >> 2) & 1) * 8;
            *reinterpret_cast<uint2*>(d) = __builtin_bit_cast(uint2, h);
            *reinterpret_cast<uint2*>(d + 16) = __builtin_bit_cast(uint2, l);
        }
        __syncthreads();
    }
    static_assert(!(PB16 != 0 && CEN != 0), "the centre rides on exact binary16 operands");
    const float ua = PB16 ? *a_unit : 0.0f, ub = PB16 ? *b_unit : 0.0f;
    for (int it = s0 + wave * iters / WAVES; it < it1; ++it) {
        RunRegs<C> rw;
        load_run_strided<C>(rw, bc + (int64_t)it * w_step, w_piece, bs + (int64_t)it * ws_step);
        if constexpr (ADENSE == 1) {
            // a ring of AHEAD operand pieces per row tile keeps the L2 round trips ahead of the MFMAs
            constexpr int AHEAD = 4;
            uint4 fa[AHEAD][TM];
#pragma unroll
            for (int m = 0; m < AHEAD; ++m)
#pragma unroll
                for (int i = 0; i < TM; ++i) fa[m][i] = ap[i][(int64_t)(it * 4 * C + m) * 64];
#pragma unroll
            for (int m = 0; m < 4 * C; ++m) {
                uint4 cur[TM];
#pragma unroll
                for (int i = 0; i < TM; ++i) cur[i] = fa[m % AHEAD][i];
                if (m + AHEAD < 4 * C) {
#pragma unroll
                    for (int i = 0; i < TM; ++i) fa[m % AHEAD][i] = ap[i][(int64_t)(it * 4 * C + m + AHEAD) * 64];
                }
                if constexpr (PB16 != 0) {
                    const bf16x8_t fw = run_operand_bf16<C>(rw, m, ub);
#pragma unroll
                    for (int i = 0; i < TM; ++i)
                        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fw, __builtin_bit_cast(bf16x8_t, cur[i]), acc[i], 0, 0, 0);
                } else {
                    const half8_t fw = run_operand<C>(rw, m);
#pragma unroll
                    for (int i = 0; i < TM; ++i)
                        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fw, __builtin_bit_cast(half8_t, cur[i]), acc[i], 0, 0, 0);
                }
            }
            continue;
        }
        RunRegs<C> ra[TM];
#pragma unroll
        for (int i = 0; i < TM; ++i) load_run_strided<C>(ra[i], ac[i] + (int64_t)it * a_step, a_piece, as[i] + (int64_t)it * as_step);
#pragma unroll
        for (int m = 0; m < 4 * C; ++m) {
            if constexpr (PB16 != 0) {
                const bf16x8_t fw = run_operand_bf16<C>(rw, m, ub);
#pragma unroll
                for (int i = 0; i < TM; ++i)
                    acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fw, run_operand_bf16<C>(ra[i], m, ua), acc[i], 0, 0, 0);
                continue;
            }
            const half8_t fb = run_operand<C>(rw, m);
            if constexpr (CEN != 0) {                          // the lane's run starts at element hi * 32 C of the iteration
                const uint4* mp = reinterpret_cast<const uint4*>(mes) + ((((it - s0) * 64 * C + hi * 32 * C) >> 3) + m) * 2 + (lane & 1);
                accm = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb, __builtin_bit_cast(half8_t, *mp), accm, 0, 0, 0);
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb, run_operand<C>(ra[i], m), acc[i], 0, 0, 0);
        }
    }
    if constexpr (PB16 == 0) {
        // tensor units (and the 2^8 * 2^8 of the scale placement)
        const float us = (*a_unit) * (*b_unit) * 65536.0f;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][e] *= us;
    }
    if constexpr (CEN != 0) {
        // the rank-one term: every output row gets W^ me.  accm[e] holds it for this lane's column n(e), split over
        // the lane pair (hi part, lo part); the expanded operand carries 2^-8, the centre 2^-4, and the tensor unit
        // is missing.  Each wave adds its own share of K to its partial accumulators, so the sum over waves (and
        // K slices) completes it.
        const float ys = (*b_unit) * 4096.0f;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const float yv = (accm[e] + __shfl_xor(accm[e], 1)) * ys;
#pragma unroll
            for (int i = 0; i < TM; ++i) acc[i][e] += yv;
        }
        __syncthreads();                                       // all waves are done with the staged centre: red is free
    }
    // bf16 low-rank extension: slices of 32 columns dealt to the waves (K slice 0 only)
    auto lowrank_into = [&](float16_t (&dst)[TM]) {
        for (int j0 = wave * 32; j0 < (slice == 0 ? r : 0); j0 += WAVES * 32) {
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const int j = j0 + q * 16 + hi * 8;
                const bf16x8_t fu = *reinterpret_cast<const bf16x8_t*>(u + (int64_t)nrow * r + j);
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    const int mrow = min(m0 + i * 32 + (lane & 31), M - 1);
                    const bf16x8_t ft = *reinterpret_cast<const bf16x8_t*>(t + (int64_t)mrow * ldt + j);
                    dst[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fu, ft, dst[i], 0, 0, 0);
                }
            }
        }
    };
    if constexpr (PB16 == 0) lowrank_into(acc);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) red[wave][i * 16 + e][lane] = acc[i][e];
    __syncthreads();
    // acc[i][e] of lane l: m = 32 i + l % 32, n = 8 (e / 4) + 4 (l / 32) + e % 4.  One (i, e / 4, l) per thread and pass.
    constexpr int NID = (TM * 256 + 64 * WAVES - 1) / (64 * WAVES);
    auto store4 = [&](int m, int n, const float (&v)[4]) {
        if (OUT_F32) {
            *reinterpret_cast<float4*>((float*)out + (int64_t)m * N + n) = make_float4(v[0], v[1], v[2], v[3]);
        } else {
            uint2 w;
            w.x = bf16_bits(v[0]) | (bf16_bits(v[1]) << 16);
            w.y = bf16_bits(v[2]) | (bf16_bits(v[3]) << 16);
            *reinterpret_cast<uint2*>((uint16_t*)out + (int64_t)m * N + n) = w;
        }
    };
    float keep[NID][4];                                        // PB16: the rounded residual (+ bias) while the low-rank term is summed
#pragma unroll
    for (int p = 0; p < NID; ++p) {
        const int id = threadIdx.x + p * 64 * WAVES;
        const int l = id & 63, g = (id >> 6) & 3, i = min(id >> 8, TM - 1);
        const int m = m0 + i * 32 + (l & 31), n = n0 + 8 * g + 4 * (l >> 5);
        float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int w = 0; w < WAVES; ++w)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] += red[w][i * 16 + 4 * g + e][l];
        const bool live = id < TM * 256 && m < M && n < N;     // N % 4 == 0 is required
        if constexpr (PB16 != 0) {
            if (!part) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[e] = rb(v[e]);                           // the reference's bf16 matmul result, then its bf16 bias add
                    if (bias && live) v[e] = rb(v[e] + bias_value(bias, bias_f32, n + e));
                }
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) keep[p][e] = v[e];
        }
        if (!live) continue;
        if (part) {                                            // binary32 partial [nsplit][M][N]; the bias waits for the sum
            *reinterpret_cast<float4*>(part + ((int64_t)slice * M + m) * N + n) = make_float4(v[0], v[1], v[2], v[3]);
            continue;
        }
        if constexpr (PB16 == 0) {
            if (bias)
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] += bias_value(bias, bias_f32, n + e);
            store4(m, n, v);
        }
    }
    if constexpr (PB16 != 0) {
        const bool low = r > 0 && slice == 0;                  // uniform over the workgroup
        const int nlw = min(WAVES, r / 32);                    // waves that hold low-rank products
        if (low) {
            __syncthreads();                                   // the residual sums have been read: red is free
            float16_t accl[TM];
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int e = 0; e < 16; ++e) accl[i][e] = 0.0f;
            lowrank_into(accl);
            if (wave < nlw) {
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int e = 0; e < 16; ++e) red[wave][i * 16 + e][lane] = accl[i][e];
            }
            __syncthreads();
        }
        if (part && !low) return;
#pragma unroll
        for (int p = 0; p < NID; ++p) {
            const int id = threadIdx.x + p * 64 * WAVES;
            const int l = id & 63, g = (id >> 6) & 3, i = min(id >> 8, TM - 1);
            const int m = m0 + i * 32 + (l & 31), n = n0 + 8 * g + 4 * (l >> 5);
            if (id >= TM * 256 || m >= M || n >= N) continue;
            float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            if (low) {
                for (int w = 0; w < nlw; ++w)
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] += red[w][i * 16 + 4 * g + e][l];
            }
            if (part) {                                        // the low-rank term of this tile: one more partial, slot nsplit
                *reinterpret_cast<float4*>(part + ((int64_t)nsplit * M + m) * N + n) = make_float4(v[0], v[1], v[2], v[3]);
                continue;
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                v[e] += keep[p][e];
                if (OUT_F32) v[e] = rb(v[e]);                  // a binary32 buffer still receives bf16 values in this mode
            }
            store4(m, n, v);
        }
    }
}

// Several weight matrices against ONE packed activation in one launch (q/k/v, gate/up): the column tiles of the
// members are laid end to end along grid x.  A decode-sized k or v projection alone is 16 workgroups and costs a
// whole launch latency; next to q it is free.
template <int TM, int C, int WAVES, int OUT_F32, int CEN = 0, int PB16 = 0, int ADENSE = 0>
__global__ __launch_bounds__(64 * WAVES) void gemm_nvfp4_skinny_grouped_kernel(
    const uint8_t* __restrict__ a_codes, const uint8_t* __restrict__ a_scales, const float* __restrict__ a_unit, int M, int K,
    const SkinnyGroup grp)
{
    const int tile = (int)blockIdx.x;
    int g = 0, start = 0;
#pragma unroll
    for (int i = 0; i + 1 < kMaxGroupMembers; ++i)
        if (i + 1 < grp.count && tile >= grp.m[i].tile_end) { g = i + 1; start = grp.m[i].tile_end; }
    // select with a uniform chain of compares rather than a dynamic index into the kernel arguments
    SkinnyMember mm = grp.m[0];
#pragma unroll
    for (int i = 1; i < kMaxGroupMembers; ++i)
        if (g == i) mm = grp.m[i];
    skinny_tile<TM, C, WAVES, OUT_F32, CEN, PB16, ADENSE>(a_codes, a_scales, a_unit, mm.b_codes, mm.b_scales, mm.b_unit, M, mm.N, K, mm.t, mm.u,
                                            mm.r, mm.bias, mm.out, mm.bias_f32, (tile - start) * 32, mm.ldt, mm.part, grp.nsplit,
                                            grp.center, mm.decode);
}

// A packed weight in the decode layout (gemm_common.h): one thread per 16-byte piece of codes, then the scale bytes.
// Derived data, built once per weight update and cached beside the packed form like the tiled expansion.
__global__ __launch_bounds__(256) void decode_weight_kernel(const uint8_t* __restrict__ codes, const uint8_t* __restrict__ scales,
                                                            int N, int K, uint8_t* __restrict__ out, int64_t blocks)
{
    const int iters = K / 256;
    for (int64_t b = blockIdx.x; b < blocks; b += gridDim.x) {
        const int tile = (int)(b / iters), it = (int)(b % iters);
        uint8_t* dst = out + b * kDecodeBlock;
        const int l = threadIdx.x & 63, j = threadIdx.x >> 6;              // lane, piece
        const int row = tile * 32 + (l & 31), h = l >> 5;
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        if (row < N) v = *reinterpret_cast<const uint4*>(codes + (int64_t)row * (K / 2) + it * 128 + h * 64 + 16 * j);
        *reinterpret_cast<uint4*>(dst + j * 1024 + l * 16) = v;
        if (j == 0) {
            uint2 sc = make_uint2(0u, 0u);
            if (row < N) sc = *reinterpret_cast<const uint2*>(scales + (int64_t)row * (K / 16) + it * 16 + h * 8);
            *reinterpret_cast<uint2*>(dst + 4096 + l * 8) = sc;
        }
    }
}

size_t decode_weight_bytes(int64_t N, int64_t K)
{
    if (N <= 0 || K <= 0 || K % 256) return 0;
    return (size_t)((N + 31) / 32) * (size_t)(K / 256) * kDecodeBlock;
}

int decode_weight(const void* codes, const void* scales, int64_t N, int64_t K, void* out, hipStream_t st)
{
    if (N <= 0 || K <= 0 || N > INT32_MAX || K > INT32_MAX) return METIS_E_ARG;
    if (K % 256) return METIS_E_SHAPE;
    if (!codes || !scales || !out || ((uintptr_t)codes % 16) || ((uintptr_t)scales % 8) || ((uintptr_t)out % 16)) return METIS_E_ARG;
    const int64_t blocks = ((N + 31) / 32) * (K / 256);
    int64_t g = blocks;
    const int64_t cap = (int64_t)device_cus() * 16;
    if (g > cap) g = cap;
    hipLaunchKernelGGL(decode_weight_kernel, dim3((unsigned)g), dim3(256), 0, st, (const uint8_t*)codes, (const uint8_t*)scales, (int)N, (int)K,
                       (uint8_t*)out, blocks);
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

// The activation of a decode-sized call as ready MFMA operands for the wide-run layout of skinny_tile (K % 256 == 0):
// piece ((row tile, iteration, m), lane) holds the 8 elements k = 256 it + 128 (lane / 32) + 8 m .. of row
// 32 tile + lane % 32, rows past M zero.  Exact mode: e2m1 * e4m3 * 2^-8 in binary16 (the tensor unit stays outside).
// PB16: the reference's bf16 value bf16(bf16(e4m3 * unit) * e2m1), and with a centre (mean mode, one bf16 value per
// column) its me + QDQ(x - me) rounded to bf16 once more (src/Metis/Metis/bitlinear.py:330-333 in bf16 arithmetic).
// DEF: the quantizer call deferred its scale bytes (nvfp4_quant.hip): `scales` holds bf16 block maxima, `partials` the
// partial tensor maxima; unit (written to unit_out) and E4M3 bytes are formed here, in the arithmetic of that call (QMODE).
// (block `block` of `nblocks`: a launch may give its first blocks to other work)
// The eight values of one piece of the rotated operand: the block's two code words c, its scale byte sb, the tensor
// unit (bf16 arithmetic), half = which eight of the block's sixteen outputs, sign_mask = the rotation's signs.
template <int PB16>
__device__ __forceinline__ uint4 rotated_operand_piece(const uint2 c, const uint32_t sb, const float unit, const int half, const uint32_t sign_mask)
{
    typedef float float2_t __attribute__((ext_vector_type(2)));
    const float dq = PB16 ? rb(e4m3_value(sb) * unit) : e4m3_value(sb) * 0.00390625f;
    const float2_t p[8] = {__builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.x, 1.0f, 0), __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.x, 1.0f, 1),
                           __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.x, 1.0f, 2), __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.x, 1.0f, 3),
                           __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.y, 1.0f, 0), __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.y, 1.0f, 1),
                           __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.y, 1.0f, 2), __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c.y, 1.0f, 3)};
    float blk[kBlock];
#pragma unroll
    for (int n = 0; n < kBlock; ++n) {
        const float x = PB16 ? rb(p[n >> 1][n & 1] * dq) : p[n >> 1][n & 1] * dq;
        // sign[n] of the rotation; inputs 8..15 change sign for the outputs 8..15 (H[n][8 + j] = -H[n][j] there)
        const uint32_t flip = (((sign_mask >> n) & 1u) ^ (n >= 8 ? (uint32_t)half : 0u)) << 31;
        blk[n] = __uint_as_float(__float_as_uint(x) ^ flip);
    }
    float o[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        float acc = blk[0];
#pragma unroll
        for (int n = 1; n < kBlock; ++n) acc = (__builtin_popcount(n & j) & 1) ? acc - blk[n] : acc + blk[n];
        o[j] = acc * 0.0625f;
    }
    uint4 v;
    if constexpr (PB16 != 0) {
        v.x = rb_pair(o[0], o[1]); v.y = rb_pair(o[2], o[3]); v.z = rb_pair(o[4], o[5]); v.w = rb_pair(o[6], o[7]);
    } else {
        const half2_t h0 = {(_Float16)o[0], (_Float16)o[1]}, h1 = {(_Float16)o[2], (_Float16)o[3]};
        const half2_t h2 = {(_Float16)o[4], (_Float16)o[5]}, h3 = {(_Float16)o[6], (_Float16)o[7]};
        v.x = __builtin_bit_cast(uint32_t, h0); v.y = __builtin_bit_cast(uint32_t, h1);
        v.z = __builtin_bit_cast(uint32_t, h2); v.w = __builtin_bit_cast(uint32_t, h3);
    }
    return v;
}

// RHT (sign_mask): the call multiplies with a weight packed in the rotated domain; see skinny_operand_rht_kernel.
template <int PB16, int DEF, int QMODE, int RHT = 0>
__device__ __forceinline__ void skinny_operand_block(int block, int nblocks, const uint32_t* __restrict__ codes,
                                                     const uint8_t* __restrict__ scales, const float* __restrict__ unit_p,
                                                     const uint16_t* __restrict__ center, int M, int K, int tiles,
                                                     uint4* __restrict__ out, const uint32_t* __restrict__ partials,
                                                     float* __restrict__ unit_out, uint32_t sign_mask = 0u)
{
    typedef float float2_t __attribute__((ext_vector_type(2)));
    const int iters = K / 256;
    const int64_t total = (int64_t)tiles * iters * 1024;
    float unit = 0.0f;
    if constexpr (DEF != 0) {
        unit = tensor_unit_of<QMODE>(fold_partial_maxima(partials));
        if (block == 0 && threadIdx.x == 0) *unit_out = unit;
    } else if constexpr (PB16 != 0) {
        unit = *unit_p;
    }
    const uint16_t* __restrict__ maxima = reinterpret_cast<const uint16_t*>(scales);
    for (int64_t idx = (int64_t)block * 256 + threadIdx.x; idx < total; idx += (int64_t)nblocks * 256) {
        const int lane = (int)(idx & 63), m = (int)((idx >> 6) & 15);
        const int64_t ti = idx >> 10;
        const int it = (int)(ti % iters), tile = (int)(ti / iters);
        const int row = tile * 32 + (lane & 31), k0 = it * 256 + (lane >> 5) * 128 + 8 * m;
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        if (row < M) {
            uint32_t sb;
            if constexpr (DEF != 0) sb = scale_byte_of<QMODE>(maxima[(int64_t)row * (K / 16) + (k0 >> 4)], unit);
            else sb = scales[(int64_t)row * (K / 16) + (k0 >> 4)];
            if constexpr (RHT != 0) {
                v = rotated_operand_piece<PB16>(reinterpret_cast<const uint2*>(codes)[(int64_t)row * (K / 16) + (k0 >> 4)], sb, unit, m & 1,
                                                sign_mask);
                out[idx] = v;
                continue;
            }
            const uint32_t c = codes[(int64_t)row * (K / 8) + (k0 >> 3)];
            if constexpr (PB16 != 0) {
                const float dq = rb(e4m3_value(sb) * unit);
                const float2_t p[4] = {__builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, 1.0f, 0), __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, 1.0f, 1),
                                       __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, 1.0f, 2), __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, 1.0f, 3)};
                float o[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) o[j] = p[j >> 1][j & 1] * dq;
                if (center) {
                    const uint4 cw = *reinterpret_cast<const uint4*>(center + k0);
                    const uint32_t cws[4] = {cw.x, cw.y, cw.z, cw.w};
#pragma unroll
                    for (int j = 0; j < 8; ++j) o[j] = ((j & 1) ? bf16_hi(cws[j >> 1]) : bf16_lo(cws[j >> 1])) + rb(o[j]);
                }
                v.x = rb_pair(o[0], o[1]); v.y = rb_pair(o[2], o[3]); v.z = rb_pair(o[4], o[5]); v.w = rb_pair(o[6], o[7]);
            } else {
                v = expand8(c, scale_pair(sb));
            }
        }
        out[idx] = v;
    }
}

template <int PB16, int DEF = 0, int QMODE = 0>
__global__ __launch_bounds__(256) void skinny_operand_kernel(const uint32_t* __restrict__ codes, const uint8_t* __restrict__ scales,
                                                             const float* __restrict__ unit_p, const uint16_t* __restrict__ center,
                                                             int M, int K, int tiles, uint4* __restrict__ out,
                                                             const uint32_t* __restrict__ partials = nullptr,
                                                             float* __restrict__ unit_out = nullptr)
{
    skinny_operand_block<PB16, DEF, QMODE>((int)blockIdx.x, (int)gridDim.x, codes, scales, unit_p, center, M, K, tiles, out, partials,
                                           unit_out);
}

// NV recipe at decode size.  The cached weight holds the codes of the ROTATED weight, and the forward multiplies with
// W~ = rotate_back(QDQ(rotate(W))) (src/Metis/Metis/bitlinear.py:577-585, 395-405): per block of 16 along K,
// W~[n] = sign[n] / 16 * sum_k H[k][n] q[k] with q the dequantized rotated block.  The decode-sized kernel streams the
// packed weight as it is, so the rotation goes to the other operand:
//     sum_n x^[n] W~[n] = sum_k q[k] a'[k],   a'[k] = 1/16 * sum_n H[n][k] (sign[n] x^[n])
// -- the activation's dequantized block rotated forward and scaled by 1/16.  The sums are exact in binary32 (sixteen
// values of one block: at most 16 significant bits), a' is rounded once to the operand's 16-bit format (the tiled
// path rounds W~ once instead).  A thread forms the eight values of its piece from the whole block (both code words).
template <int PB16, int DEF, int QMODE>
__global__ __launch_bounds__(256) void skinny_operand_rht_kernel(const uint2* __restrict__ codes, const uint8_t* __restrict__ scales,
                                                                 const float* __restrict__ unit_p, int M, int K, int tiles,
                                                                 uint4* __restrict__ out, const uint32_t* __restrict__ partials,
                                                                 float* __restrict__ unit_out, uint32_t sign_mask)
{
    skinny_operand_block<PB16, DEF, QMODE, 1>((int)blockIdx.x, (int)gridDim.x, reinterpret_cast<const uint32_t*>(codes), scales, unit_p,
                                              nullptr, M, K, tiles, out, partials, unit_out, sign_mask);
}

// One launch for the two small independent steps between a decode-sized layer's quantizer and its GEMM: the first
// `finish_blocks` blocks finish the rank-r projection (lowrank_small_steps.h), the others build the activation's
// operands from a tensor whose quantizer call deferred its scale bytes.
template <int PB16, int QMODE, int RHT = 0>
__global__ __launch_bounds__(256) void decode_prepare_kernel(int finish_blocks, const float* __restrict__ lr_ws, int chunks, int MR, int R,
                                                             const uint16_t* __restrict__ s, uint16_t* __restrict__ xv,
                                                             uint16_t* __restrict__ t, const uint32_t* __restrict__ codes,
                                                             const uint8_t* __restrict__ maxima, const uint16_t* __restrict__ center,
                                                             int M, int K, int tiles, uint4* __restrict__ out,
                                                             const uint32_t* __restrict__ partials, float* __restrict__ unit_out,
                                                             uint32_t sign_mask)
{
    if ((int)blockIdx.x < finish_blocks) {
        lowrank_small_finish_block((int)blockIdx.x, lr_ws, chunks, MR, R, s, xv, t);
        return;
    }
    skinny_operand_block<PB16, 1, QMODE, RHT>((int)blockIdx.x - finish_blocks, (int)gridDim.x - finish_blocks, codes, maxima, nullptr, center,
                                              M, K, tiles, out, partials, unit_out, sign_mask);
}

size_t skinny_operand_bytes(int64_t M, int64_t K)
{
    if (M <= 0 || K <= 0) return 0;
    return (size_t)((M + 63) / 64) * 64 * (size_t)K * 2;      // whole pairs of 32-row tiles
}

int skinny_operand(const void* codes, const void* scales, const float* unit, int64_t M, int64_t K, int mode, const void* center,
                   void* out, hipStream_t st)
{
    if (mode == METIS_MODE_P32_F32) mode = METIS_MODE_P32;
    if (mode != METIS_MODE_P32 && mode != METIS_MODE_PB16) return METIS_E_ARG;
    if (M <= 0 || M >= 256 || K <= 0 || K % 256 || K > INT32_MAX) return METIS_E_SHAPE;
    if (!codes || !scales || !out || ((uintptr_t)codes % 4) || ((uintptr_t)out % 16) || ((uintptr_t)center % 16)) return METIS_E_ARG;
    if (mode == METIS_MODE_PB16 ? !unit : center != nullptr) return METIS_E_ARG;   // a centre belongs to bf16 arithmetic
    const int tiles = (int)((M + 63) / 64) * 2;
    const int64_t total = (int64_t)tiles * (K / 256) * 1024;
    const int g = (int)((total + 255) / 256);
    if (mode == METIS_MODE_PB16)
        hipLaunchKernelGGL(skinny_operand_kernel<1>, dim3(g), dim3(256), 0, st, (const uint32_t*)codes, (const uint8_t*)scales, unit,
                           (const uint16_t*)center, (int)M, (int)K, tiles, (uint4*)out);
    else
        hipLaunchKernelGGL(skinny_operand_kernel<0>, dim3(g), dim3(256), 0, st, (const uint32_t*)codes, (const uint8_t*)scales, unit,
                           (const uint16_t*)center, (int)M, (int)K, tiles, (uint4*)out);
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

int skinny_operand_deferred(const void* codes, const void* deferred, int64_t M, int64_t K, int qmode, int mode, const void* center,
                            float* unit_out, void* out, hipStream_t st)
{
    if (mode == METIS_MODE_P32_F32) mode = METIS_MODE_P32;
    if ((mode != METIS_MODE_P32 && mode != METIS_MODE_PB16) || (qmode != METIS_MODE_P32 && qmode != METIS_MODE_PB16)) return METIS_E_ARG;
    if (M <= 0 || M >= 256 || K <= 0 || K % 256 || K > INT32_MAX) return METIS_E_SHAPE;
    if (!codes || !unit_out || !out || ((uintptr_t)codes % 4) || ((uintptr_t)out % 16) || ((uintptr_t)center % 16)) return METIS_E_ARG;
    if (center && mode != METIS_MODE_PB16) return METIS_E_ARG;
    Workspace ws;
    if (const int rc = carve_deferred(const_cast<void*>(deferred), deferred_bytes(M, K), M, K, &ws)) return rc;
    const int tiles = (int)((M + 63) / 64) * 2;
    const int64_t total = (int64_t)tiles * (K / 256) * 1024;
    const int g = (int)((total + 255) / 256);
#define METIS_SOD(P, Q) hipLaunchKernelGGL((skinny_operand_kernel<P, 1, Q>), dim3(g), dim3(256), 0, st, (const uint32_t*)codes, \
                                           (const uint8_t*)ws.amax, nullptr, (const uint16_t*)center, (int)M, (int)K, tiles, (uint4*)out, \
                                           (const uint32_t*)ws.gmax, unit_out)
    if (mode == METIS_MODE_PB16) { if (qmode) METIS_SOD(1, 1); else METIS_SOD(1, 0); }
    else { if (qmode) METIS_SOD(0, 1); else METIS_SOD(0, 0); }
#undef METIS_SOD
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

// The operand of a decode-sized call against a ROTATED packed weight (NV recipe): the activation's dequantized blocks
// rotated forward and scaled by 1/16 (skinny_operand_rht_kernel).  deferred = nullptr: scale bytes and unit as given;
// otherwise the quantizer call deferred them (qmode = its arithmetic) and unit receives the tensor unit.
int skinny_operand_rht(const void* codes, const void* scales, float* unit, const void* deferred, int64_t M, int64_t K, int qmode, int mode,
                       uint32_t sign_mask, void* out, hipStream_t st)
{
    if (mode == METIS_MODE_P32_F32) mode = METIS_MODE_P32;
    if (mode != METIS_MODE_P32 && mode != METIS_MODE_PB16) return METIS_E_ARG;
    if (sign_mask > 0xffffu) return METIS_E_ARG;
    if (M <= 0 || M >= 256 || K <= 0 || K % 256 || K > INT32_MAX) return METIS_E_SHAPE;
    if (!codes || !out || ((uintptr_t)codes % 8) || ((uintptr_t)out % 16)) return METIS_E_ARG;
    const int tiles = (int)((M + 63) / 64) * 2;
    const int64_t total = (int64_t)tiles * (K / 256) * 1024;
    const int g = (int)((total + 255) / 256);
    if (deferred) {
        if ((qmode != METIS_MODE_P32 && qmode != METIS_MODE_PB16) || !unit) return METIS_E_ARG;
        Workspace ws;
        if (const int rc = carve_deferred(const_cast<void*>(deferred), deferred_bytes(M, K), M, K, &ws)) return rc;
#define METIS_SOR(P, Q) hipLaunchKernelGGL((skinny_operand_rht_kernel<P, 1, Q>), dim3(g), dim3(256), 0, st, (const uint2*)codes, \
                                           (const uint8_t*)ws.amax, nullptr, (int)M, (int)K, tiles, (uint4*)out, (const uint32_t*)ws.gmax, \
                                           unit, sign_mask)
        if (mode == METIS_MODE_PB16) { if (qmode) METIS_SOR(1, 1); else METIS_SOR(1, 0); }
        else { if (qmode) METIS_SOR(0, 1); else METIS_SOR(0, 0); }
#undef METIS_SOR
        return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
    }
    if (!scales || (mode == METIS_MODE_PB16 && !unit)) return METIS_E_ARG;
    if (mode == METIS_MODE_PB16)
        hipLaunchKernelGGL((skinny_operand_rht_kernel<1, 0, 0>), dim3(g), dim3(256), 0, st, (const uint2*)codes, (const uint8_t*)scales, unit,
                           (int)M, (int)K, tiles, (uint4*)out, nullptr, nullptr, sign_mask);
    else
        hipLaunchKernelGGL((skinny_operand_rht_kernel<0, 0, 0>), dim3(g), dim3(256), 0, st, (const uint2*)codes, (const uint8_t*)scales, unit,
                           (int)M, (int)K, tiles, (uint4*)out, nullptr, nullptr, sign_mask);
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

// lowrank_small + skinny_operand_deferred on the same activation (x [M, K] bf16 and its packed form) in two launches
// instead of three: partial sums of the projection, then one launch that finishes it and builds the operands.
// x = nullptr: the first of the two already ran beside the quantizer (quantize_row_deferred_partial): one launch.
int decode_prepare_deferred(const void* x, int64_t ldx, const void* v, int64_t R, const void* s, void* xv, void* t, void* workspace,
                            size_t workspace_bytes, const void* codes, const void* deferred, int64_t M, int64_t K, int qmode, int mode,
                            const void* center, float* unit_out, void* out, hipStream_t st, int rotate, uint32_t sign_mask)
{
    if (mode == METIS_MODE_P32_F32) mode = METIS_MODE_P32;
    if (rotate && (center || sign_mask > 0xffffu || ((uintptr_t)codes % 8))) return METIS_E_ARG;   // a rotated operand: uncentred, whole blocks per load
    if ((mode != METIS_MODE_P32 && mode != METIS_MODE_PB16) || (qmode != METIS_MODE_P32 && qmode != METIS_MODE_PB16)) return METIS_E_ARG;
    if (M <= 0 || M >= 256 || K <= 0 || K % 256 || K > INT32_MAX) return METIS_E_SHAPE;
    if (!codes || !unit_out || !out || ((uintptr_t)codes % 4) || ((uintptr_t)out % 16) || ((uintptr_t)center % 16)) return METIS_E_ARG;
    if (center && mode != METIS_MODE_PB16) return METIS_E_ARG;
    Workspace ws;
    if (const int rc = carve_deferred(const_cast<void*>(deferred), deferred_bytes(M, K), M, K, &ws)) return rc;
    int chunks = 0;
    if (x) {
        if (const int rc = lowrank_small_partial(x, ldx, v, M, R, K, s, xv, t, workspace, workspace_bytes, st, &chunks)) return rc;
    } else {
        // the partial sums are in the workspace already (quantize_row_deferred_partial on the same shapes)
        if (R <= 0 || R % 32 || R > 128) return METIS_E_SHAPE;
        if (!xv || (t && !s) || ((uintptr_t)xv % 8) || ((uintptr_t)t % 8) || ((uintptr_t)s % 2)) return METIS_E_ARG;
        if (!workspace || ((uintptr_t)workspace % 16) || workspace_bytes < lowrank_small_workspace_bytes(M, R, K)) return METIS_E_WORKSPACE;
        int kc;
        chunks = lowrank_small_chunks(K, &kc);
    }
    const int fb = lowrank_small_finish_blocks(M, R);
    const int tiles = (int)((M + 63) / 64) * 2;
    const int64_t total = (int64_t)tiles * (K / 256) * 1024;
    const int g = fb + (int)((total + 255) / 256);
#define METIS_DP(P, Q, H) hipLaunchKernelGGL((decode_prepare_kernel<P, Q, H>), dim3(g), dim3(256), 0, st, fb, (const float*)workspace, chunks, \
                                             (int)(M * R), (int)R, (const uint16_t*)s, (uint16_t*)xv, (uint16_t*)t, (const uint32_t*)codes, \
                                             (const uint8_t*)ws.amax, (const uint16_t*)center, (int)M, (int)K, tiles, (uint4*)out, \
                                             (const uint32_t*)ws.gmax, unit_out, sign_mask)
#define METIS_DPH(P, Q) do { if (rotate) METIS_DP(P, Q, 1); else METIS_DP(P, Q, 0); } while (0)
    if (mode == METIS_MODE_PB16) { if (qmode) METIS_DPH(1, 1); else METIS_DPH(1, 0); }
    else { if (qmode) METIS_DPH(0, 1); else METIS_DPH(0, 0); }
#undef METIS_DPH
#undef METIS_DP
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

// Adds the K slices of the skinny kernel in ascending order, then bias and output conversion.
// grid (column quads / 256, M, members).
// PB16: the slices hold the residual product only; their sum is rounded to bf16, the bias added in bf16, then the
// low-rank term (slot nsplit, members with r > 0) and the final rounding.
template <int OUT_F32, int PB16 = 0>
__global__ __launch_bounds__(256) void skinny_splitk_reduce_kernel(const SkinnyGroup grp, int M)
{
    SkinnyMember mm = grp.m[0];
#pragma unroll
    for (int i = 1; i < kMaxGroupMembers; ++i)
        if ((int)blockIdx.z == i) mm = grp.m[i];
    const int n = 4 * (int)(blockIdx.x * 256u + threadIdx.x), m = (int)blockIdx.y;
    if (n >= mm.N) return;
    const float* src = mm.part + (int64_t)m * mm.N + n;
    float4 v = *reinterpret_cast<const float4*>(src);
    for (int z = 1; z < grp.nsplit; ++z) {
        const float4 p = *reinterpret_cast<const float4*>(src + (int64_t)z * M * mm.N);
        v.x += p.x; v.y += p.y; v.z += p.z; v.w += p.w;
    }
    if constexpr (PB16 != 0) {
        v.x = rb(v.x); v.y = rb(v.y); v.z = rb(v.z); v.w = rb(v.w);
        if (mm.bias) {
            v.x = rb(v.x + bias_value(mm.bias, mm.bias_f32, n));     v.y = rb(v.y + bias_value(mm.bias, mm.bias_f32, n + 1));
            v.z = rb(v.z + bias_value(mm.bias, mm.bias_f32, n + 2)); v.w = rb(v.w + bias_value(mm.bias, mm.bias_f32, n + 3));
        }
        if (mm.r > 0) {
            const float4 p = *reinterpret_cast<const float4*>(src + (int64_t)grp.nsplit * M * mm.N);
            v.x += p.x; v.y += p.y; v.z += p.z; v.w += p.w;
        }
        if (OUT_F32) { v.x = rb(v.x); v.y = rb(v.y); v.z = rb(v.z); v.w = rb(v.w); }
    } else if (mm.bias) {
        v.x += bias_value(mm.bias, mm.bias_f32, n);     v.y += bias_value(mm.bias, mm.bias_f32, n + 1);
        v.z += bias_value(mm.bias, mm.bias_f32, n + 2); v.w += bias_value(mm.bias, mm.bias_f32, n + 3);
    }
    if (OUT_F32) {
        *reinterpret_cast<float4*>((float*)mm.out + (int64_t)m * mm.N + n) = v;
    } else {
        uint2 w;
        w.x = bf16_bits(v.x) | (bf16_bits(v.y) << 16);
        w.y = bf16_bits(v.z) | (bf16_bits(v.w) << 16);
        *reinterpret_cast<uint2*>((uint16_t*)mm.out + (int64_t)m * mm.N + n) = w;
    }
}

static int launch_skinny_reduce(const SkinnyGroup& grp, int64_t M, int out_dtype, hipStream_t st, bool pb16 = false)
{
    int nmax = 0;
    for (int i = 0; i < grp.count; ++i) nmax = grp.m[i].N > nmax ? grp.m[i].N : nmax;
    const dim3 rgrid((unsigned)((nmax / 4 + 255) / 256), (unsigned)M, (unsigned)grp.count);
    if (pb16) {
        if (out_dtype == METIS_DTYPE_F32)
            hipLaunchKernelGGL((skinny_splitk_reduce_kernel<1, 1>), rgrid, dim3(256), 0, st, grp, (int)M);
        else
            hipLaunchKernelGGL((skinny_splitk_reduce_kernel<0, 1>), rgrid, dim3(256), 0, st, grp, (int)M);
    } else if (out_dtype == METIS_DTYPE_F32)
        hipLaunchKernelGGL(skinny_splitk_reduce_kernel<1>, rgrid, dim3(256), 0, st, grp, (int)M);
    else
        hipLaunchKernelGGL(skinny_splitk_reduce_kernel<0>, rgrid, dim3(256), 0, st, grp, (int)M);
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

template <int TM, int C, int WAVES>
static int launch_skinny_grouped(const void* a_codes, const void* a_scales, const float* a_unit, int64_t M, int64_t K,
                                 const SkinnyGroup& grp, int tiles, int out_dtype, hipStream_t st, bool pb16, bool adense)
{
    const bool split = grp.nsplit > 1;
    const dim3 grid((unsigned)tiles, (unsigned)((M + 32 * TM - 1) / (32 * TM)), (unsigned)(split ? grp.nsplit : 1)), block(64 * WAVES);
    if constexpr (C == 4) {
        if (adense) {                                          // the activation as ready operands (skinny_operand)
            if (grp.center) return METIS_E_ARG;
#define METIS_SKD(O, P) hipLaunchKernelGGL((gemm_nvfp4_skinny_grouped_kernel<TM, C, WAVES, O, 0, P, 1>), grid, block, 0, st, \
                                           (const uint8_t*)a_codes, (const uint8_t*)a_scales, a_unit, (int)M, (int)K, grp)
            if (pb16) { if (out_dtype == METIS_DTYPE_F32) METIS_SKD(1, 1); else METIS_SKD(0, 1); }
            else { if (out_dtype == METIS_DTYPE_F32) METIS_SKD(1, 0); else METIS_SKD(0, 0); }
#undef METIS_SKD
            if (hipGetLastError() != hipSuccess) return METIS_E_LAUNCH;
            return split ? launch_skinny_reduce(grp, M, out_dtype, st, pb16) : METIS_OK;
        }
    }
    if (adense) return METIS_E_ARG;
    if constexpr (C == 4) {
        if (grp.a_decode) {                                    // the packed activation in the decode layout: exact, centred or bf16 evaluation
#define METIS_SKA(O, CE, P) hipLaunchKernelGGL((gemm_nvfp4_skinny_grouped_kernel<TM, C, WAVES, O, CE, P, 2>), grid, block, 0, st, \
                                               (const uint8_t*)a_codes, (const uint8_t*)a_scales, a_unit, (int)M, (int)K, grp)
            const bool f32 = out_dtype == METIS_DTYPE_F32;
            if (pb16) { if (grp.center) return METIS_E_ARG; if (f32) METIS_SKA(1, 0, 1); else METIS_SKA(0, 0, 1); }
            else if (grp.center) { if (f32) METIS_SKA(1, 1, 0); else METIS_SKA(0, 1, 0); }
            else { if (f32) METIS_SKA(1, 0, 0); else METIS_SKA(0, 0, 0); }
#undef METIS_SKA
            if (hipGetLastError() != hipSuccess) return METIS_E_LAUNCH;
            return split ? launch_skinny_reduce(grp, M, out_dtype, st, pb16) : METIS_OK;
        }
    }
    if (grp.a_decode) return METIS_E_ARG;
    if (pb16) {                                                // the reference's all-bf16 evaluation
        if (grp.center) return METIS_E_ARG;
        if (out_dtype == METIS_DTYPE_F32)
            hipLaunchKernelGGL((gemm_nvfp4_skinny_grouped_kernel<TM, C, WAVES, 1, 0, 1>), grid, block, 0, st, (const uint8_t*)a_codes,
                               (const uint8_t*)a_scales, a_unit, (int)M, (int)K, grp);
        else
            hipLaunchKernelGGL((gemm_nvfp4_skinny_grouped_kernel<TM, C, WAVES, 0, 0, 1>), grid, block, 0, st, (const uint8_t*)a_codes,
                               (const uint8_t*)a_scales, a_unit, (int)M, (int)K, grp);
        if (hipGetLastError() != hipSuccess) return METIS_E_LAUNCH;
        return split ? launch_skinny_reduce(grp, M, out_dtype, st, true) : METIS_OK;
    }
    if constexpr (C == 4) {
        if (grp.center) {                                      // mean mode (wide runs only)
            if (out_dtype == METIS_DTYPE_F32)
                hipLaunchKernelGGL((gemm_nvfp4_skinny_grouped_kernel<TM, C, WAVES, 1, 1>), grid, block, 0, st, (const uint8_t*)a_codes,
                                   (const uint8_t*)a_scales, a_unit, (int)M, (int)K, grp);
            else
                hipLaunchKernelGGL((gemm_nvfp4_skinny_grouped_kernel<TM, C, WAVES, 0, 1>), grid, block, 0, st, (const uint8_t*)a_codes,
                                   (const uint8_t*)a_scales, a_unit, (int)M, (int)K, grp);
            if (hipGetLastError() != hipSuccess) return METIS_E_LAUNCH;
            return split ? launch_skinny_reduce(grp, M, out_dtype, st) : METIS_OK;
        }
    }
    if (grp.center) return METIS_E_ARG;
    if (out_dtype == METIS_DTYPE_F32)
        hipLaunchKernelGGL((gemm_nvfp4_skinny_grouped_kernel<TM, C, WAVES, 1>), grid, block, 0, st, (const uint8_t*)a_codes,
                           (const uint8_t*)a_scales, a_unit, (int)M, (int)K, grp);
    else
        hipLaunchKernelGGL((gemm_nvfp4_skinny_grouped_kernel<TM, C, WAVES, 0>), grid, block, 0, st, (const uint8_t*)a_codes,
                           (const uint8_t*)a_scales, a_unit, (int)M, (int)K, grp);
    if (hipGetLastError() != hipSuccess) return METIS_E_LAUNCH;
    return split ? launch_skinny_reduce(grp, M, out_dtype, st) : METIS_OK;
}

// K slices for the skinny kernel when its column tiles would leave compute units idle: enough to put two
// workgroups on every unit, every wave of every slice keeping at least two iterations, at most 8.  1 = no split.
static int skinny_split_factor(int64_t tiles, int64_t K, int c)
{
    const int cus = device_cus();
    if (cus <= 0 || tiles <= 0 || tiles >= cus) return 1;
    int64_t s = 2 * (int64_t)cus / tiles;
    const int64_t iters = K / (64 * c);
    if (s > iters / 16) s = iters / 16;
    if (s > 8) s = 8;
    return s < 1 ? 1 : (int)s;
}

// Workspace for the partial sums of a grouped call ([slices + 1][M][N] binary32 per member: bf16 arithmetic keeps the
// low-rank term in a slot of its own); 0 = K is not split.
size_t gemm_grouped_workspace_bytes(int64_t M, int64_t K, const GemmMember* members, int count)
{
    if (!members || count < 1 || M <= 0 || M >= 256 || K <= 0 || K % 64) return 0;
    int64_t tiles = 0, ntot = 0;
    for (int i = 0; i < count; ++i) {
        if (members[i].N <= 0) return 0;
        tiles += (members[i].N + 31) / 32;
        ntot += members[i].N;
    }
    const int s1 = skinny_split_factor(tiles, K, 1), s4 = K % 256 == 0 ? skinny_split_factor(tiles, K, 4) : 1;
    const int s = s1 > s4 ? s1 : s4;                        // which run width applies depends on pointer alignment
    return s <= 1 ? 0 : (size_t)(s + 1) * (size_t)M * (size_t)ntot * sizeof(float);
}

// One activation against up to four weight matrices.  Shapes the skinny kernel does not take fall back to one
// gemm_nvfp4 call per member (same results either way).
// Shape chosen for a grouped call on the skinny kernel: run width, row tiles per wave, waves, K slices.
struct SkinnyShape {
    int c, tm, waves, nsplit;
};
static SkinnyShape skinny_shape(int64_t M, int64_t K, int64_t tiles, bool al8, bool have_workspace)
{
    // Shape heuristics from measurements at 3584/4608/18944-wide projections: wide runs whenever alignment
    // allows; two row tiles per wave when M > 32 unless that leaves fewer workgroups than half the CUs (then the
    // row tiles go to separate workgroups); four waves per workgroup only when there are plenty of
    // workgroups anyway.
    SkinnyShape s;
    s.c = (K % 256 == 0 && al8) ? 4 : 1;
    s.nsplit = (have_workspace && !measure_env("METIS_GEMM_NOSPLIT")) ? skinny_split_factor(tiles, K, s.c) : 1;
    s.tm = (M <= 32 || tiles * s.nsplit < device_cus() / 2) ? 1 : 2;
    s.waves = (s.tm == 1 && M <= 32 && tiles >= 2 * device_cus()) ? 4 : 8;
    return s;
}
// mean mode inside the skinny kernel: wide runs, and the workgroup's slice of the centre must fit the LDS reduction buffer
static bool skinny_center_fits(const SkinnyShape& s, int64_t K)
{
    const int64_t iters = K / (64 * s.c), slice = ((iters + s.nsplit - 1) / s.nsplit) * 64 * s.c;
    return s.c == 4 && slice <= (int64_t)s.waves * s.tm * 16 * 64;
}

// 1 when a grouped call of this shape can take a centre (mean mode in one pass over the weights), else 0: the caller
// then adds W^ me as a binary32 bias computed with packed_gemv.  Scale-byte pointers are assumed 8-byte aligned.
int gemm_grouped_center_supported(int64_t M, int64_t K, const GemmMember* members, int count, int have_workspace)
{
    if (!members || count < 1 || count > 4 || M <= 0 || M >= 256 || K <= 0 || K % 64 || measure_env("METIS_GEMM_SMALL")) return 0;
    int64_t tiles = 0;
    for (int i = 0; i < count; ++i) {
        if (members[i].N <= 0 || members[i].N % 4) return 0;
        tiles += (members[i].N + 31) / 32;
    }
    return skinny_center_fits(skinny_shape(M, K, tiles, true, have_workspace != 0), K) ? 1 : 0;
}

int gemm_nvfp4_grouped(const void* a_codes, const void* a_scales, const float* a_unit, int64_t M, int64_t K,
                       const GemmMember* members, int count, int out_dtype, hipStream_t st, void* workspace,
                       size_t workspace_bytes, const float* center, bool pb16, bool a_dense)
{
    if (!members || count < 1) return METIS_E_ARG;
    if ((uintptr_t)center % 16) return METIS_E_ARG;
    if ((pb16 || a_dense) && center) return METIS_E_ARG;
    if (a_dense && (K % 256 || !a_unit)) return METIS_E_ARG;
    // no scale-byte pointer: a_codes is the packed activation in the decode layout (decode_weight applied to it)
    const bool a_decode = !a_dense && a_codes && !a_scales;
    if (a_decode && (K % 256 || M >= 256)) return METIS_E_ARG;
    if (a_dense || a_decode) a_scales = a_codes;              // unused by the kernel: the checks below see an aligned pointer
    bool skinny = M > 0 && M < 256 && K % 64 == 0 && count <= kMaxGroupMembers && !measure_env("METIS_GEMM_SMALL") &&
                  a_codes && a_scales && a_unit && !((uintptr_t)a_codes % 16) && !((uintptr_t)a_scales % 2) && K <= INT32_MAX &&
                  (out_dtype == METIS_DTYPE_BF16 || out_dtype == METIS_DTYPE_F32);
    bool al8 = ((uintptr_t)a_scales % 8) == 0;
    int64_t tiles = 0, ntot = 0;
    for (int i = 0; i < count && skinny; ++i) {
        const GemmMember& g = members[i];
        if ((!g.b_decode && (!g.b_codes || !g.b_scales)) || ((uintptr_t)g.b_decode % 16) || (g.b_decode && K % 256) || !g.b_unit || !g.out || g.N <= 0 || g.N > INT32_MAX || g.N % 4 || g.r < 0 || g.r % 32 ||
            (g.r > 0 && (!g.t || !g.u)) || (g.ldt != 0 && (g.ldt < g.r || g.ldt % 8 || g.ldt > INT32_MAX)) || ((uintptr_t)g.b_codes % 16) || ((uintptr_t)g.b_scales % 2) || ((uintptr_t)g.out % 16) ||
            ((uintptr_t)g.t % 16) || ((uintptr_t)g.u % 16) || ((uintptr_t)g.bias % (g.bias_is_f32 ? 4 : 2)))
            skinny = false;
        al8 = al8 && (g.b_decode || ((uintptr_t)g.b_scales % 8) == 0);
        tiles += (g.N + 31) / 32;
        ntot += g.N;
    }
    if (!skinny || tiles > INT32_MAX) {
        for (int i = 0; i < count; ++i)
            if (!members[i].b_codes || !members[i].b_scales) return METIS_E_ARG;   // only the decode-sized kernel reads the decode layout
        if (center || pb16 || a_dense || a_decode) return METIS_E_ARG;     // the centre, the bf16 evaluation, ready operands and the decode layout are only taken by the single-launch path
        for (int i = 0; i < count; ++i) {
            const GemmMember& g = members[i];
            if (g.ldt != 0 && g.ldt != g.r) return METIS_E_ARG;   // a strided t is only taken by the single-launch path
            const int rc = gemm_nvfp4(a_codes, a_scales, a_unit, g.b_codes, g.b_scales, g.b_unit, M, g.N, K, g.t, g.u, g.r, g.bias,
                                      g.out, out_dtype, st, nullptr, 0, g.bias_is_f32 != 0);
            if (rc != METIS_OK) return rc;
        }
        return METIS_OK;
    }
    const SkinnyShape shape = skinny_shape(M, K, tiles, al8, workspace != nullptr);
    int c = shape.c, nsplit = shape.nsplit, tm = shape.tm, waves = shape.waves;
    if (const char* f = measure_env("METIS_SKINNY_SHAPE")) {        // measurement switch: "tm,c,waves,slices"
        int ftm = 0, fc = 0, fw = 0, fs = 0;
        if (sscanf(f, "%d,%d,%d,%d", &ftm, &fc, &fw, &fs) == 4 && (ftm == 1 || ftm == 2) && (fc == 1 || (fc == 4 && c == 4)) &&
            (fw == 4 || fw == 8) && fs >= 1 && fs <= 8 && (fs == 1 || workspace) && K / (64 * fc) >= fs) {
            tm = ftm; c = fc; waves = fw; nsplit = fs;
        }
    }
    if ((a_dense || a_decode) && c != 4) return METIS_E_ARG;   // weight scale bytes must be 8-byte aligned for wide runs
    const size_t slots = (size_t)nsplit + (pb16 ? 1 : 0);      // bf16 arithmetic: one more for the low-rank term
    if (nsplit > 1 && (((uintptr_t)workspace % 16) || workspace_bytes < slots * (size_t)M * (size_t)ntot * sizeof(float)))
        return METIS_E_WORKSPACE;
    if (center && !skinny_center_fits(SkinnyShape{c, tm, waves, nsplit}, K)) return METIS_E_ARG;
    SkinnyGroup grp = {};
    grp.count = count;
    grp.nsplit = nsplit;
    grp.center = center;
    grp.a_decode = a_decode ? 1 : 0;
    int end = 0;
    float* part = (float*)workspace;
    for (int i = 0; i < count; ++i) {
        const GemmMember& g = members[i];
        end += (int)((g.N + 31) / 32);
        const bool dec = g.b_decode && c == 4;
        if (!dec && (!g.b_codes || !g.b_scales)) return METIS_E_ARG;
        grp.m[i] = SkinnyMember{(const uint8_t*)(dec ? g.b_decode : g.b_codes), (const uint8_t*)g.b_scales, g.b_unit, (const uint16_t*)g.t,
                                (const uint16_t*)g.u, (const uint16_t*)g.bias, g.out, nsplit > 1 ? part : nullptr, (int)g.N,
                                (int)g.r, end, g.bias_is_f32 != 0, (int)(g.ldt ? g.ldt : g.r), dec ? 1 : 0};
        part += slots * (size_t)M * (size_t)g.N;
    }
#define METIS_SKG(TM, C, W) return launch_skinny_grouped<TM, C, W>(a_codes, a_scales, a_unit, M, K, grp, (int)tiles, out_dtype, st, pb16, a_dense)
    if (tm == 1) {
        if (waves == 4) { if (c == 4) METIS_SKG(1, 4, 4); else METIS_SKG(1, 1, 4); }
        else { if (c == 4) METIS_SKG(1, 4, 8); else METIS_SKG(1, 1, 8); }
    } else {
        if (waves == 4) { if (c == 4) METIS_SKG(2, 4, 4); else METIS_SKG(2, 1, 4); }
        else { if (c == 4) METIS_SKG(2, 4, 8); else METIS_SKG(2, 1, 8); }
    }
#undef METIS_SKG
}

// The single-matrix call is a group of one.
static int gemm_skinny(const void* a_codes, const void* a_scales, const float* a_unit, const void* b_codes,
                       const void* b_scales, const float* b_unit, int64_t M, int64_t N, int64_t K, const void* t,
                       const void* u, int64_t r, const void* bias, void* out, int out_dtype, hipStream_t st, int bias_f32,
                       void* workspace, size_t workspace_bytes)
{
    const GemmMember g = {b_codes, b_scales, b_unit, t, u, r, bias, out, N, bias_f32, 0, nullptr};
    return gemm_nvfp4_grouped(a_codes, a_scales, a_unit, M, K, &g, 1, out_dtype, st, workspace, workspace_bytes, nullptr);
}

// ---------------------------------------------------------------------------------------------
// Expansion of a packed tensor to binary16: value = e2m1(code) * e4m3(scale) * 2^-8, exact.
// One thread per 8 elements (one dword of codes -> 16 bytes).  HBM-bound: 0.5625 B read, 2 B written
// per element.  The expanded tensor is what gemm_f16_large_kernel consumes; it is derived data that
// callers may cache next to the packed weight (the reference caches the dequantized weight the
// same way, src/Metis/Metis/bitlinear.py:563-589).
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void expand_f16_kernel(const uint32_t* __restrict__ codes, const uint8_t* __restrict__ scales,
                                                         uint4* __restrict__ out, int64_t noct)
{
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < noct; i += (int64_t)gridDim.x * 256)
        out[i] = expand8(codes[i], scale_pair(scales[i >> 1]));
}

int expand_f16(const void* codes, const void* scales, int64_t rows, int64_t cols, void* out, hipStream_t st)
{
    if (rows < 0 || cols < 0) return METIS_E_ARG;
    if (cols % kBlock) return METIS_E_SHAPE;
    const int64_t noct = rows * cols / 8;
    if (noct == 0) return METIS_OK;
    if (!codes || !scales || !out || ((uintptr_t)codes % 4) || ((uintptr_t)out % 16)) return METIS_E_ARG;
    int64_t g = (noct + 255) / 256;
    const int64_t cap = (int64_t)device_cus() * 16;
    if (g > cap) g = cap;
    hipLaunchKernelGGL(expand_f16_kernel, dim3((int)g), dim3(256), 0, st, (const uint32_t*)codes, (const uint8_t*)scales,
                       (uint4*)out, noct);
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

// ---------------------------------------------------------------------------------------------
// GEMM on expanded operands: same tile (256 x 256, 8 waves of 128 x 64, K step 64), same epilogue, but
// the inner loop is MFMA + LDS reads only.  Operand tiles go HBM/L2 -> LDS directly
// (global_load_lds_dwordx4, no registers, no VALU), one full step ahead, into a double buffer of
// 2 x 64 KiB.  LDS rows are 128 bytes with the 16-byte chunk index XOR-ed by (row & 7): the 8
// lanes of one LDS access phase hit 8 different chunk columns, so fragment reads are conflict
// free without padding (a direct load fills 1 KiB of contiguous LDS, which rules padding out).
// ---------------------------------------------------------------------------------------------
constexpr int X_STAGE_BYTES = (L_BM + L_BN) * BK * 2;             // 64 KiB: 512 rows x 128 B

template <int OUT_F32>
__global__ __launch_bounds__(512, 1) void gemm_f16_large_kernel(
    const uint16_t* __restrict__ a_exp, const float* __restrict__ a_unit, const uint16_t* __restrict__ b_exp,
    const float* __restrict__ b_unit, int M, int N, int K, const uint16_t* __restrict__ t, const uint16_t* __restrict__ u,
    int r, const uint16_t* __restrict__ bias, void* __restrict__ out, int tiles_m, int tiles_n)
{
    extern __shared__ __attribute__((aligned(1024))) uint8_t xlds[];
    constexpr int TM = 4, TN = 2, WTN = 64;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 2, wn = wave & 3;

    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) / 8;
    const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (logical >= total) return;
    constexpr int GM = 4;
    const int group = logical / (GM * tiles_n);
    const int first_m = group * GM;
    const int gsize = min(tiles_m - first_m, GM);
    const int tm = first_m + (logical % (GM * tiles_n)) % gsize;
    const int tn = (logical % (GM * tiles_n)) / gsize;
    const int m0 = tm * L_BM, n0 = tn * L_BN;

    float16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    // ---- async staging: instruction j of wave w fills LDS rows (j*8 + w)*8 .. +7 (1 KiB); lane -> (row, chunk)
    const uint8_t* src[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int trow = (j * 8 + wave) * 8 + (lane >> 3);          // row of the A|B tile, 0..511
        const int chunk = (lane & 7) ^ (trow & 7);                  // logical 16-byte chunk that belongs at this slot
        const bool is_a = trow < L_BM;
        const int64_t grow = is_a ? min(m0 + trow, M - 1) : min(n0 + trow - L_BM, N - 1);
        src[j] = reinterpret_cast<const uint8_t*>((is_a ? a_exp : b_exp) + grow * K) + chunk * 16;
    }
    auto stage_in = [&](int buf, int k0) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
            __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)(src[j] + (int64_t)k0 * 2),
                                             (void __attribute__((address_space(3)))*)(xlds + buf * X_STAGE_BYTES + (j * 8 + wave) * 1024),
                                             16, 0, 0);
    };

    const int steps = K / BK;
    stage_in(0, 0);
    if (steps > 1) {
        stage_in(1, BK);
        __builtin_amdgcn_s_waitcnt(0x0F78);                         // vmcnt(8): the first step has landed, the second may fly
    } else {
        __builtin_amdgcn_s_waitcnt(0x0F70);                         // vmcnt(0)
    }
    __syncthreads();

    // fragment addressing: row = base + (lane & 31), chunk = 2*ks + (lane >> 5), slot = chunk ^ (row & 7)
    const int frow = lane & 31, fhi = lane >> 5;
    int a_row_off[TM], b_row_off[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) a_row_off[i] = (wm * 128 + i * 32 + frow) * 128;
#pragma unroll
    for (int j = 0; j < TN; ++j) b_row_off[j] = (L_BM + wn * WTN + j * 32 + frow) * 128;
    const int sw = frow & 7;                                        // (row & 7): tile bases are multiples of 32
    half8_t fa[2][TM], fb[2][TN];
    auto load_frags = [&](int fbuf, int buf, int ks) {
        const int slot = ((2 * ks + fhi) ^ sw) * 16;
        const uint8_t* base = xlds + buf * X_STAGE_BYTES + slot;
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[fbuf][i] = *reinterpret_cast<const half8_t*>(base + a_row_off[i]);
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[fbuf][j] = *reinterpret_cast<const half8_t*>(base + b_row_off[j]);
    };
    auto mfmas = [&](int fbuf) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[fbuf][j], fa[fbuf][i], acc[i][j], 0, 0, 0);
    };

    load_frags(0, 0, 0);
    for (int s = 0; s < steps; ++s) {
        const int buf = s & 1;
        load_frags(1, buf, 1);
        mfmas(0);
        load_frags(0, buf, 2);
        mfmas(1);
        load_frags(1, buf, 3);
        mfmas(0);
        // every wave has issued its last reads of `buf`; the loads of step s+1 (issued one step ago) must have landed
        __builtin_amdgcn_s_waitcnt(0x0070);                         // vmcnt(0), lgkmcnt(0)
        __syncthreads();
        if (s + 2 < steps) stage_in(buf, (s + 2) * BK);             // refill the buffer just released
        if (s + 1 < steps) load_frags(0, buf ^ 1, 0);
        mfmas(1);
    }
    __syncthreads();

    const float us = (*a_unit) * (*b_unit) * 65536.0f;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] *= us;

    // ---- bf16 low-rank extension, 32 columns per step: rows staged through registers, padded 144-byte rows
    uint16_t* plds = reinterpret_cast<uint16_t*>(xlds);
    for (int j0 = 0; j0 < r; j0 += 32) {
        {
            const bool is_a = tid < L_BM;
            const int64_t grow = is_a ? min(m0 + tid, M - 1) : min(n0 + tid - L_BM, N - 1);
            const uint4* sp = reinterpret_cast<const uint4*>((is_a ? t : u) + grow * r + j0);
            uint4* dp = reinterpret_cast<uint4*>(plds + tid * L_STRIDE);
#pragma unroll
            for (int c = 0; c < 4; ++c) dp[c] = sp[c];
        }
        __syncthreads();
        const int foff = frow * L_STRIDE + fhi * 8;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            bf16x8_t ga[TM], gb[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) ga[i] = *reinterpret_cast<const bf16x8_t*>(plds + (wm * 128 + i * 32) * L_STRIDE + foff + ks * 16);
#pragma unroll
            for (int j = 0; j < TN; ++j) gb[j] = *reinterpret_cast<const bf16x8_t*>(plds + (L_BM + wn * WTN + j * 32) * L_STRIDE + foff + ks * 16);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gb[j], ga[i], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = m0 + wm * 128 + i * 32 + (lane & 31);
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = n0 + wn * WTN + j * 32 + 8 * g + 4 * (lane >> 5);
                if (n >= N) continue;
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

int gemm_expanded(const void* a_exp, const float* a_unit, const void* b_exp, const float* b_unit, int64_t M, int64_t N,
                  int64_t K, const void* t, const void* u, int64_t r, const void* bias, void* out, int out_dtype,
                  hipStream_t st)
{
    if (M < 0 || N < 0 || K < 0 || r < 0) return METIS_E_ARG;
    if (out_dtype != METIS_DTYPE_BF16 && out_dtype != METIS_DTYPE_F32) return METIS_E_ARG;
    if (K % kBlock) return METIS_E_SHAPE;
    if (K % BK || K == 0 || N % 4 || r % 32 || (r > 0 && (!t || !u))) return METIS_E_ARG;
    if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return METIS_E_ARG;
    if (M == 0 || N == 0) return METIS_OK;
    if (!a_exp || !a_unit || !b_exp || !b_unit || !out) return METIS_E_ARG;
    if (((uintptr_t)a_exp % 16) || ((uintptr_t)b_exp % 16) || ((uintptr_t)out % 16)) return METIS_E_ARG;
    static bool attr_set[2][64] = {};
    const size_t lds_bytes = 2 * (size_t)X_STAGE_BYTES;
    const int f32 = out_dtype == METIS_DTYPE_F32;
    const void* fn = f32 ? (const void*)gemm_f16_large_kernel<1> : (const void*)gemm_f16_large_kernel<0>;
    if (const int rc = allow_dynamic_lds(fn, lds_bytes, attr_set[f32])) return rc;
    const int tiles_m = (int)((M + L_BM - 1) / L_BM), tiles_n = (int)((N + L_BN - 1) / L_BN);
    const int total = tiles_m * tiles_n;
    const unsigned grid_x = (unsigned)(((total + 7) / 8) * 8);
    const uint16_t *ae = (const uint16_t*)a_exp, *be = (const uint16_t*)b_exp, *tp = (const uint16_t*)t,
                   *up = (const uint16_t*)u, *bp = (const uint16_t*)bias;
    int Mi = (int)M, Ni = (int)N, Ki = (int)K, ri = (int)r, tmi = tiles_m, tni = tiles_n;
    void* args[] = {&ae, &a_unit, &be, &b_unit, &Mi, &Ni, &Ki, &tp, &up, &ri, &bp, &out, &tmi, &tni};
    if (hipLaunchKernel(fn, dim3(grid_x), dim3(512), args, lds_bytes, st) != hipSuccess) {
        (void)hipGetLastError();
        return METIS_E_LAUNCH;
    }
    return METIS_OK;
}

int gemm_nvfp4(const void* a_codes, const void* a_scales, const float* a_unit, const void* b_codes, const void* b_scales,
               const float* b_unit, int64_t M, int64_t N, int64_t K, const void* t, const void* u, int64_t r,
               const void* bias, void* out, int out_dtype, hipStream_t st, void* workspace, size_t workspace_bytes,
               int bias_f32)
{
    if (!a_codes || !a_scales || !a_unit || !b_codes || !b_scales || !b_unit || !out) return METIS_E_ARG;
    if (M < 0 || N < 0 || K < 0 || r < 0) return METIS_E_ARG;
    if (out_dtype != METIS_DTYPE_BF16 && out_dtype != METIS_DTYPE_F32) return METIS_E_ARG;
    if (K % kBlock) return METIS_E_SHAPE;
    if (N % 4 || r % 32 || (r > 0 && (!t || !u))) return METIS_E_ARG;
    if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return METIS_E_ARG;
    if (((uintptr_t)a_codes % 16) || ((uintptr_t)b_codes % 16) || ((uintptr_t)a_scales % 2) || ((uintptr_t)b_scales % 2) ||
        ((uintptr_t)out % 16) || ((uintptr_t)t % 16) || ((uintptr_t)u % 16) || ((uintptr_t)bias % (bias_f32 ? 4 : 2)))
        return METIS_E_ARG;
    if (K % 32) return METIS_E_ARG;                            // 16-byte code chunks: rows must stay 16-byte aligned
    if (M == 0 || N == 0) return METIS_OK;
    if (M >= 256 && N >= 256 && K % BK == 0 && !measure_env("METIS_GEMM_SMALL")) {
#ifdef METIS_MEASURE
        if (measure_env("METIS_GEMM_W4"))                      // 4 waves of 128 x 128: measured 15 % slower than 8 of 128 x 64
            return launch_large<2>(a_codes, a_scales, a_unit, b_codes, b_scales, b_unit, M, N, K, t, u, r, bias, out, out_dtype, st, bias_f32);
#endif
        SplitPlan plan = {1, 0};
        if (workspace && !measure_env("METIS_GEMM_NOSPLIT")) {
            plan = split_plan(M, N, K);
            if (plan.nsplit > 1 && (((uintptr_t)workspace % 16) || workspace_bytes < gemm_workspace_bytes(M, N, K))) return METIS_E_WORKSPACE;
        }
        return launch_large<4>(a_codes, a_scales, a_unit, b_codes, b_scales, b_unit, M, N, K, t, u, r, bias, out, out_dtype, st,
                               bias_f32, (float*)workspace, plan.nsplit, plan.nfull);
    }
    if (M < 256 && K % 64 == 0 && !measure_env("METIS_GEMM_SMALL"))    // up to four 64-row passes over the weights beat a mostly empty 256-row tile
        return gemm_skinny(a_codes, a_scales, a_unit, b_codes, b_scales, b_unit, M, N, K, t, u, r, bias, out, out_dtype, st, bias_f32,
                           workspace, workspace_bytes);
    constexpr int BM = 128, BN = 128;
    dim3 grid((unsigned)((N + BN - 1) / BN), (unsigned)((M + BM - 1) / BM));
    if (out_dtype == METIS_DTYPE_F32)
        hipLaunchKernelGGL((gemm_nvfp4_kernel<BM, BN, 1>), grid, dim3(256), 0, st, (const uint8_t*)a_codes,
                           (const uint8_t*)a_scales, a_unit, (const uint8_t*)b_codes, (const uint8_t*)b_scales, b_unit,
                           (int)M, (int)N, (int)K, (const uint16_t*)t, (const uint16_t*)u, (int)r, (const uint16_t*)bias, out, bias_f32);
    else
        hipLaunchKernelGGL((gemm_nvfp4_kernel<BM, BN, 0>), grid, dim3(256), 0, st, (const uint8_t*)a_codes,
                           (const uint8_t*)a_scales, a_unit, (const uint8_t*)b_codes, (const uint8_t*)b_scales, b_unit,
                           (int)M, (int)N, (int)K, (const uint16_t*)t, (const uint16_t*)u, (int)r, (const uint16_t*)bias, out, bias_f32);
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

}  // namespace metis
