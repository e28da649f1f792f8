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
#include <stdlib.h>

namespace metis {

// swz(q) for row q of a tile (bits b1, b2, b3 of the row number): slot bit 0 = b2, slot bit 1 = b1 ^ b3.
// Any 8 consecutive rows then cover 8 different 16-byte units of a 128-byte bank period, and any 16
// consecutive rows 16 different units of a 256-byte period.
__host__ __device__ __forceinline__ int xt_swz(int q) { return ((q >> 2) & 1) | ((((q >> 1) ^ (q >> 3)) & 1) << 1); }

// ---------------------------------------------------------------------------------------------
// packed NVFP4 -> tiled binary16.  One wave per tile: lane l writes slot l (row l / 4).  A wave walks
// eight consecutive k tiles of one tile row, so the 128-byte lines of codes it touches are used whole.
// HBM-bound: 0.5625 B read, 2 B written per element.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void expand_xt_kernel(const uint32_t* __restrict__ codes, const uint8_t* __restrict__ scales,
                                                        uint4* __restrict__ out, int rows, int K, int row_tiles)
{
    const int lane = threadIdx.x & 63;
    const int kt = K / 32, kgroups = (kt + 7) / 8;
    const int q = lane >> 2, chunk = (lane & 3) ^ xt_swz(q);
    const int64_t nunits = (int64_t)row_tiles * kgroups;
    for (int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); unit < nunits; unit += (int64_t)gridDim.x * 4) {
        const int rb = (int)(unit / kgroups), kg = (int)(unit - (int64_t)rb * kgroups);
        const int row = rb * 16 + q;
        const bool live = row < rows;
        const int kend = min(kt, kg * 8 + 8);
        for (int kb = kg * 8; kb < kend; ++kb) {
            uint4 v = make_uint4(0u, 0u, 0u, 0u);
            if (live) {
                const int k8 = kb * 4 + chunk;                   // index of the 8-element chunk inside the row
                v = expand8(codes[(int64_t)row * (K / 8) + k8], scale_pair(scales[(int64_t)row * (K / 16) + (k8 >> 1)]));
            }
            out[((int64_t)rb * kt + kb) * 64 + lane] = v;
        }
    }
}

size_t expand_xt_bytes(int64_t rows, int64_t cols)
{
    if (rows <= 0 || cols <= 0) return 0;
    return (size_t)((rows + 15) / 16) * 16 * (size_t)cols * 2;
}

int expand_xt(const void* codes, const void* scales, int64_t rows, int64_t cols, void* out, hipStream_t st)
{
    if (rows < 0 || cols < 0) return METIS_E_ARG;
    if (cols % kBlock) return METIS_E_SHAPE;
    if (cols % 32 || rows > INT32_MAX - 16 || cols > INT32_MAX) return METIS_E_ARG;
    if (rows == 0 || cols == 0) return METIS_OK;
    if (!codes || !scales || !out || ((uintptr_t)codes % 4) || ((uintptr_t)out % 16)) return METIS_E_ARG;
    const int row_tiles = (int)((rows + 15) / 16);
    const int64_t units = (int64_t)row_tiles * ((cols / 32 + 7) / 8);
    int64_t g = (units + 3) / 4;
    const int64_t cap = (int64_t)device_cus() * 16;
    if (g > cap) g = cap;
    hipLaunchKernelGGL(expand_xt_kernel, dim3((unsigned)g), dim3(256), 0, st, (const uint32_t*)codes, (const uint8_t*)scales,
                       (uint4*)out, (int)rows, (int)cols, row_tiles);
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

// ---------------------------------------------------------------------------------------------
// The GEMM.  256 x 256 per workgroup; WN_WAVES = 4: eight waves (2 x 4) of 128 x 64, two per SIMD;
// WN_WAVES = 2: four waves (2 x 2) of 128 x 128, one per SIMD (a third less LDS read traffic).
// A stage is 32 k of the A|B tile: 32 KiB = 32 operand tiles, one direct load each.  NS slots of KS stages form a
// ring (shipped: three slots of one stage, 96 KiB).  Iteration s (stage s in slot s % NS):
//     read fragments (s, k 16..31)            | MFMAs on fragments (s, k 0..15)
//     wait: own fragment reads done, own loads of stage s+1 landed;  BARRIER
//     issue loads of stage s+NS into slot s % NS (every wave holds what it needs of stage s in registers)
//     read fragments (s+1, k 0..15)           | MFMAs on fragments (s, k 16..31)
// so a stage's loads have NS-1 iterations to arrive and the waits never drain the queue.
// ---------------------------------------------------------------------------------------------
constexpr int XT_STAGE = 32 * 1024;

__host__ __device__ constexpr int waitcnt_imm(int vm, int lgkm)
{
    return (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | ((lgkm & 15) << 8);
}
#define METIS_WAIT(VM, LGKM) __builtin_amdgcn_s_waitcnt(waitcnt_imm(VM, LGKM))

template <int OUT_F32, int WN_WAVES, int NS, int KS = 1, int ILV = 0>
__global__ __launch_bounds__(128 * WN_WAVES, 1) void gemm_xt_kernel(
    const uint8_t* __restrict__ a_xt, const float* __restrict__ a_unit, const uint8_t* __restrict__ b_xt,
    const float* __restrict__ b_unit, int M, int N, int K, const uint16_t* __restrict__ t, const uint16_t* __restrict__ u,
    int r, const uint16_t* __restrict__ bias, void* __restrict__ out, int tiles_m, int tiles_n, int bias_f32)
{
    extern __shared__ __attribute__((aligned(1024))) uint8_t xlds[];
    constexpr int TM = 4, TN = 8 / WN_WAVES, WTN = 256 / WN_WAVES;
    constexpr int NWAVES = 2 * WN_WAVES, NTHREADS = 64 * NWAVES;
    constexpr int LPW = 32 / NWAVES;                            // direct loads per wave per stage: 4 or 8
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN_WAVES, wn = wave % WN_WAVES;

    // tile assignment: contiguous range per XCD, groups of four tile rows (see tile_origin)
    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) / 8;
    const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (logical >= total) return;
    int m0, n0;
    tile_origin(logical, tiles_m, tiles_n, m0, n0);

    float16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    // ---- direct loads: instruction j of wave w copies operand tile j * NWAVES + w of the stage (0..15 A, 16..31 B).
    // Written as assembly: the compiler orders every later LDS read behind ALL outstanding direct loads (it cannot
    // tell the ring slots apart), which would drain the queue each iteration; the waits are placed by hand instead.
    const int kt = K / 32;
    const int a_rt = (M + 15) / 16, b_rt = (N + 15) / 16;
    const uint8_t* src[LPW];                                    // wave-uniform: first byte of the tile row (k tile 0)
#pragma unroll
    for (int j = 0; j < LPW; ++j) {
        const int ot = j * NWAVES + wave;
        const bool is_a = ot < 16;
        const int rt = is_a ? min(m0 / 16 + ot, a_rt - 1) : min(n0 / 16 + ot - 16, b_rt - 1);
        src[j] = (is_a ? a_xt : b_xt) + (int64_t)rt * kt * 1024;
    }
    const uint32_t lane16 = lane * 16;
    constexpr int SLOT = KS * XT_STAGE;                         // a ring slot holds the KS stages of one iteration
    constexpr int LPS = LPW * KS;                               // direct loads per wave per slot
    auto issue_one = [&](int slot, int it, int n) {             // load n (0 .. LPS-1) of iteration `it` into `slot`
        const int sub = n / LPW, j = n % LPW;
        const uint8_t* g = src[j] + ((int64_t)it * KS + sub) * 1024;
        const uint32_t dst = (uint32_t)(slot * SLOT + sub * XT_STAGE + (j * NWAVES + wave) * 1024);   // LDS byte address of the tile
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :: "v"(lane16), "s"(g), "s"(dst) : "memory");
    };
    auto issue = [&](int slot, int it) {
#pragma unroll
        for (int n = 0; n < LPS; ++n) issue_one(slot, it, n);
    };

    // ---- fragment addressing: lane -> row lr of a 32-row MFMA tile, k half hi; chunk = 2 * ks + hi.
    // ks = 1 flips bit 1 of the chunk index, which flips bit 1 of the slot: byte offset ^ 32.
    const int lr = lane & 31, hi = lane >> 5;
    const int lane_off = (lr >> 4) * 1024 + (lr & 15) * 64 + ((hi ^ xt_swz(lr & 15)) * 16);
    const int a_off[2] = {wm * 8 * 1024 + lane_off, wm * 8 * 1024 + (lane_off ^ 32)};
    const int b_off[2] = {(16 + wn * (WTN / 16)) * 1024 + lane_off, (16 + wn * (WTN / 16)) * 1024 + (lane_off ^ 32)};
    half8_t fa[2][TM], fb[2][TN];
    auto load_frags = [&](int slot, int q) {                    // sub-step q of the slot: stage q / 2, k half q % 2; buffer q % 2
        const int x = slot * SLOT + (q >> 1) * XT_STAGE;
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[q & 1][i] = *reinterpret_cast<const half8_t*>(xlds + (a_off[q & 1] + x) + i * 2048);
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[q & 1][j] = *reinterpret_cast<const half8_t*>(xlds + (b_off[q & 1] + x) + j * 2048);
    };
    auto mfmas = [&](int fbuf) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[fbuf][j], fa[fbuf][i], acc[i][j], 0, 0, 0);
    };
    constexpr int NM = TM * TN, NF = TM + TN;
    constexpr int QL = 2 * KS - 1;                              // last sub-step of an iteration

    const int steps = kt / KS;                                  // iterations (the host picks KS = 1 unless KS divides K / 32)
    // prologue: fill the ring
#pragma unroll
    for (int p = 0; p < NS; ++p)
        if (p < steps) issue(p, p);
    if (steps >= NS) METIS_WAIT((NS - 1) * LPS, 15);
    else METIS_WAIT(0, 15);
    __syncthreads();
    load_frags(0, 0);

    // the sub-steps before the barrier: fragments of sub-step q+1 are read while the MFMAs of sub-step q run
    auto head = [&](int slot) {
#pragma unroll
        for (int q = 0; q < QL; ++q) {
            load_frags(slot, q + 1);
            mfmas(q & 1);
            sched_substep<NM, 0, NF, 0>();
        }
    };
    int s = 0, slot = 0;
    // steady state: the iteration NS ahead exists, so every wait allows NS-2 slots in flight
    for (; s + NS < steps; ++s) {
        const int nslot = slot + 1 == NS ? 0 : slot + 1;
        head(slot);
        METIS_WAIT((NS - 2) * LPS, 0);                          // own loads of iteration s+1 landed, own fragment reads of s done
        __syncthreads();
        if constexpr (ILV != 0) {
            // the direct loads are spread between the MFMAs of the last sub-step instead of issued in one burst
            load_frags(nslot, 0);
            constexpr int PER = (NM + LPS - 1) / LPS;
#pragma unroll
            for (int m = 0; m < NM; ++m) {
                if (m % PER == 0 && m / PER < LPS) issue_one(slot, s + NS, m / PER);
                const int i = m / TN, j = m % TN;
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[1][j], fa[1][i], acc[i][j], 0, 0, 0);
            }
        } else {
            issue(slot, s + NS);
            load_frags(nslot, 0);
            mfmas(1);
            sched_substep<NM, 0, NF, 0>();
        }
        slot = nslot;
    }
    // drain: nothing left to issue; the loads still in flight are at most NS-1 slots
    for (; s < steps; ++s) {
        const int nslot = slot + 1 == NS ? 0 : slot + 1;
        head(slot);
        const int ahead = steps - 2 - s;                           // iterations issued beyond s+1
        bool waited = false;
        if constexpr (NS > 3) {
            if (ahead >= NS - 3) { METIS_WAIT((NS - 3) * LPS, 0); waited = true; }
        }
        if constexpr (NS > 4) {
            if (!waited && ahead == NS - 4) { METIS_WAIT((NS - 4) * LPS, 0); waited = true; }
        }
        if (!waited) METIS_WAIT(0, 0);
        __syncthreads();
        if (s + 1 < steps) load_frags(nslot, 0);
        mfmas(1);
        sched_substep<NM, 0, NF, 0>();
        slot = nslot;
    }
    __syncthreads();                                            // the ring is free for the epilogue

    // ---- tensor units (and the 2^8 * 2^8 of the scale placement)
    const float us = (*a_unit) * (*b_unit) * 65536.0f;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] *= us;

    // ---- bf16 low-rank extension, 32 columns of T / U per step, staged in rows of 144 bytes
    uint16_t* plds = reinterpret_cast<uint16_t*>(xlds);
    const int frag_off = lr * L_STRIDE + hi * 8;
    for (int j0 = 0; j0 < r; j0 += 32) {
        for (int trow = tid; trow < L_BM + L_BN; trow += NTHREADS) {
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

    // ---- epilogue.  acc[i][j][e] of lane l: m = 32 i + l % 32, n = 32 j + 8 (e / 4) + 4 (l / 32) + e % 4 in the wave tile.
    if constexpr (!OUT_F32) {
        if ((N & 7) == 0) {
            // bf16: each wave transposes its tile through its own slice of LDS, 64 rows at a time, so that a store
            // instruction writes whole 16-byte pieces of rows (WTN * 2 contiguous bytes per row)
            constexpr int CROW = WTN + 8;                       // halves per staged row: 144 or 272 bytes
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

template <int OUT_F32, int WN_WAVES, int NS, int KS = 1, int ILV = 0>
static int launch_xt(const void* a_xt, const float* a_unit, const void* b_xt, const float* b_unit, int64_t M, int64_t N, int64_t K,
                     const void* t, const void* u, int64_t r, const void* bias, int bias_f32, void* out, hipStream_t st)
{
    static bool attr_set[64] = {};
    const void* fn = (const void*)gemm_xt_kernel<OUT_F32, WN_WAVES, NS, KS, ILV>;
    const size_t lds_bytes = (size_t)NS * KS * XT_STAGE;
    if (const int rc = allow_dynamic_lds(fn, lds_bytes, attr_set)) return rc;
    const int tiles_m = (int)((M + L_BM - 1) / L_BM), tiles_n = (int)((N + L_BN - 1) / L_BN);
    const int total = tiles_m * tiles_n;
    const unsigned grid_x = (unsigned)(((total + 7) / 8) * 8);
    const uint8_t *ae = (const uint8_t*)a_xt, *be = (const uint8_t*)b_xt;
    const uint16_t *tp = (const uint16_t*)t, *up = (const uint16_t*)u, *bp = (const uint16_t*)bias;
    int Mi = (int)M, Ni = (int)N, Ki = (int)K, ri = (int)r, tmi = tiles_m, tni = tiles_n;
    void* args[] = {&ae, &a_unit, &be, &b_unit, &Mi, &Ni, &Ki, &tp, &up, &ri, &bp, &out, &tmi, &tni, &bias_f32};
    if (hipLaunchKernel(fn, dim3(grid_x), dim3(128 * WN_WAVES), args, lds_bytes, st) != hipSuccess) {
        (void)hipGetLastError();
        return METIS_E_LAUNCH;
    }
    return METIS_OK;
}

int gemm_xt(const void* a_xt, const float* a_unit, const void* b_xt, const float* b_unit, int64_t M, int64_t N, int64_t K,
            const void* t, const void* u, int64_t r, const void* bias, int bias_f32, void* out, int out_dtype, hipStream_t st,
            int variant)
{
    if (M < 0 || N < 0 || K < 0 || r < 0) return METIS_E_ARG;
    if (out_dtype != METIS_DTYPE_BF16 && out_dtype != METIS_DTYPE_F32) return METIS_E_ARG;
    if (K % kBlock) return METIS_E_SHAPE;
    if (K % 32 || K == 0 || N % 4 || r % 32 || (r > 0 && (!t || !u))) return METIS_E_ARG;
    if (M > INT32_MAX - 256 || N > INT32_MAX - 256 || K > INT32_MAX) return METIS_E_ARG;
    if (M == 0 || N == 0) return METIS_OK;
    if (!a_xt || !a_unit || !b_xt || !b_unit || !out) return METIS_E_ARG;
    if (((uintptr_t)a_xt % 16) || ((uintptr_t)b_xt % 16) || ((uintptr_t)out % 16) || ((uintptr_t)t % 16) || ((uintptr_t)u % 16) ||
        ((uintptr_t)bias % (bias_f32 ? 4 : 2)))
        return METIS_E_ARG;
    const int f32 = out_dtype == METIS_DTYPE_F32;
#define METIS_XT(W, S) (f32 ? launch_xt<1, W, S>(a_xt, a_unit, b_xt, b_unit, M, N, K, t, u, r, bias, bias_f32, out, st) \
                            : launch_xt<0, W, S>(a_xt, a_unit, b_xt, b_unit, M, N, K, t, u, r, bias, bias_f32, out, st))
#ifdef METIS_MEASURE
#define METIS_XTK(W, S, KS_, I) (f32 ? launch_xt<1, W, S, KS_, I>(a_xt, a_unit, b_xt, b_unit, M, N, K, t, u, r, bias, bias_f32, out, st) \
                                     : launch_xt<0, W, S, KS_, I>(a_xt, a_unit, b_xt, b_unit, M, N, K, t, u, r, bias, bias_f32, out, st))
    if (variant == 5 && K % 64 == 0) return METIS_XTK(4, 2, 2, 0);
    if (variant == 6 && K % 64 == 0) return METIS_XTK(4, 2, 2, 1);
    if (variant == 7) return METIS_XTK(4, 3, 1, 1);
    if (variant == 8 && K % 64 == 0) return METIS_XTK(2, 2, 2, 0);
#undef METIS_XTK
    if (variant == 1) return METIS_XT(4, 5);
    if (variant == 2) return METIS_XT(2, 4);
    if (variant == 3) return METIS_XT(2, 5);
    if (variant == 4) return METIS_XT(4, 3);
#endif
    (void)variant;
    // measured at 8192 x 14336 x 4096: ring depths 3, 4 and 5 are within 1 % of each other (latency is covered), so the
    // smallest ring is used; spreading the direct loads between the MFMAs gains 1-2 %; two stages per barrier and
    // four waves of 128 x 128 are slower (3 % and 17 %)
    return f32 ? launch_xt<1, 4, 3, 1, 1>(a_xt, a_unit, b_xt, b_unit, M, N, K, t, u, r, bias, bias_f32, out, st)
               : launch_xt<0, 4, 3, 1, 1>(a_xt, a_unit, b_xt, b_unit, M, N, K, t, u, r, bias, bias_f32, out, st);
#undef METIS_XT
}

}  // namespace metis
