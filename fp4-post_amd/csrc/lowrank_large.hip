// Rank-r products of the low-rank branch at training / prefill sizes (256 rows and more), bf16 operands, binary32
// accumulation on MFMA.  Both are bound by one pass over the tall operand in HBM.
//
//   lowrank_nt:  xv[M, R] = x[M, K] . v[R, K]^T,  t = bf16(xv * s)      `vlinear(x)` and `torch.mul(self.s, y)` of
//                BitLinear.forward with the bf16 V of the north-star formula (src/Metis/Metis/bitlinear.py:752-756);
//                with v = U^T also dY . U of the backward pass
//   lowrank_tn:  out[C, R] = sum_l a[l, C] . b[l, R]                     the two products of the backward pass that
//                contract over tokens: dY^T . (xv * s) -> grad of U, x^T . g_xv -> grad of V (written transposed)
//
// lowrank_nt: a workgroup owns 32 rows of x and walks K in steps of 256.  The x rows (32 x 512 B) and the R rows of v
// (R x 512 B, from L2 after the first workgroup touched them) are fetched two steps ahead into registers, 16 bytes
// per thread and load, and staged in LDS with 528-byte rows; wave w multiplies the w-th quarter (64 k) of the step
// for all R columns, and the four partial sums meet in LDS at the end.
//
// lowrank_tn: the contraction runs down the rows of both operands, so each has to be turned: a workgroup owns 64
// columns of a and one slice of the tokens; a step of 64 tokens is loaded row by row (coalesced) and staged in LDS as it
// is; the MFMA fragments (8 consecutive tokens of one column) are read with the transposing LDS read of gfx950.  Token
// slices give every compute unit work; their binary32 partial results go to a caller workspace and a second kernel adds
// them in slice order.
#include "metis_device.h"
#include "metis_host.h"
#include "nvfp4_encode.h"

namespace metis {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int NT_STEP = 256;                     // k per step of lowrank_nt
constexpr int NT_STRIDE = NT_STEP + 8;           // halves per staged row: 528 bytes, conflict-free 16-byte reads

// K slices: with 32 rows per workgroup a tensor of a few thousand rows gives one workgroup per compute unit, too few
// bytes in flight to cover the memory latency.  gridDim.y workgroups then share a row tile, each walking its own range
// of steps; their binary32 partial sums go to a caller workspace ([slice][row][R]) and lowrank_nt_finish_kernel adds
// them in slice order.  One slice: the result is written directly.
//
// QMODE >= 0: the same pass also quantizes x (round to nearest, rows; METIS_MODE_P32 or _PB16 arithmetic).  The workgroup
// then has four more waves that take no part in the product: after the barrier that publishes a staged step they read
// the x rows back from LDS, two blocks of 16 per thread, and encode them while the first four waves wait for the next
// loads -- E2M1 codes, the block maximum parked as bf16, one partial tensor maximum per workgroup: what
// quant_codes_contig_kernel leaves for a consumer that forms the scale bytes itself.  (Encoding in the loading waves
// themselves put the encoder's ~250 vector instructions per step between their wait and their barrier.)
// EW = false: the loading waves encode the block they fetched themselves, one step later (kept in px), after the next
// loads are issued: 256 threads and fewer registers per workgroup, so two workgroups fit a compute unit -- the better
// form when there are more row tiles than compute units (16384 rows: 41 against 46 us; 8192 rows: 38 against 30 us).
template <int RT, int QMODE = -1, bool EW = false>  // R / 32 column tiles: 1, 2 or 4
__global__ __launch_bounds__((QMODE >= 0 && EW) ? 512 : 256) void lowrank_nt_kernel(
    const uint16_t* __restrict__ x, int64_t ldx, const uint16_t* __restrict__ v, const uint16_t* __restrict__ s,
    uint16_t* __restrict__ xv, uint16_t* __restrict__ t, int M, int K, float* __restrict__ part, uint2* __restrict__ codes,
    uint16_t* __restrict__ q_amax, uint32_t* __restrict__ q_gmax, uint32_t fill_to, int rotate)
{
    constexpr int R = RT * 32;
    constexpr int TILE_BYTES = (32 + R) * NT_STRIDE * 2;        // one staged step: x rows, then v rows
    constexpr int RED_BYTES = 4 * RT * 16 * 64 * 4;
    constexpr int LDS_BYTES = TILE_BYTES > RED_BYTES ? TILE_BYTES : RED_BYTES;
    __shared__ __attribute__((aligned(16))) unsigned char lds[LDS_BYTES];     // the staged step, then the four partial sums
    uint16_t* tile = reinterpret_cast<uint16_t*>(lds);
    float* red = reinterpret_cast<float*>(lds);                 // [wave][j][e][lane]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m0 = blockIdx.x * 32;
    const int steps_all = (K + NT_STEP - 1) / NT_STEP;          // K % 64 == 0; a short last step is padded with zeros
    const int per = (steps_all + (int)gridDim.y - 1) / (int)gridDim.y;
    const int first = (int)blockIdx.y * per, steps = max(0, min(steps_all, first + per) - first);
    __shared__ float smax[4];
    // Every row tile starts at a different step of its K range and wraps around: at any moment the workgroups then read
    // different column stripes of x instead of the same one.  With rows a multiple of 4 KiB long, 512-byte pieces at the
    // same offset of every row can fall on the same few memory channels (flushed caches, 8192 x 14336: 146 -> 104 us on one
    // machine, 126 -> 107 us on another; 8192 x 4096: 39 -> 31 us on the first, no change on the second; row lengths like
    // 7168 or 17920 bytes are indifferent).  The binary32 sums of a tile are therefore added in an order that depends on
    // the tile, the same for every call and for both forms of the kernel.
    const int rot = (rotate && steps > 0) ? (int)((blockIdx.x * (unsigned)rotate) % (unsigned)steps) : 0;
    auto kof = [&](int st) { int q = st + rot; if (q >= steps) q -= steps; return (first + q) * NT_STEP; };
    if constexpr (QMODE >= 0 && EW) {
        if (tid >= 256) {                                       // the encoding waves: same barriers as the others, nothing else shared
            const int et = tid - 256;
            float gmax = 0.0f;
            for (int st = 0; st < steps; ++st) {
                __syncthreads();                                // the step is staged
                uint4 b[2][2];
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const int id = i * 256 + et, row = id >> 4, blk = id & 15;
                    b[i][0] = *reinterpret_cast<const uint4*>(tile + row * NT_STRIDE + blk * 16);
                    b[i][1] = *reinterpret_cast<const uint4*>(tile + row * NT_STRIDE + blk * 16 + 8);
                }
                __syncthreads();                                // the tile may be overwritten: the blocks are in registers
                const int k0 = kof(st);
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const int id = i * 256 + et, row = id >> 4, k = k0 + (id & 15) * 16;
                    if (m0 + row < M && k < K) {
                        float val[kBlock];
                        const float none[kBlock] = {};
                        unpack16(b[i][0], b[i][1], val);
                        const float am = block_amax(val);
                        gmax = fmaxf(gmax, am);
                        const int64_t ib = (int64_t)(m0 + row) * (K / kBlock) + k / kBlock;
                        q_amax[ib] = (uint16_t)(__float_as_uint(am) >> 16);
                        codes[ib] = encode_block<QMODE < 0 ? 0 : QMODE, false>(val, block_scalar<QMODE < 0 ? 0 : QMODE>(am), none);
                    }
                }
            }
            // one partial maximum per workgroup, indexed over the whole grid; unused entries cleared for the folding reader
            const float wm = wave_max(gmax);
            if (lane == 0) smax[wave - 4] = wm;
            __syncthreads();                                    // the barrier the other waves pass after parking their sums
            const uint32_t gid = blockIdx.y * gridDim.x + blockIdx.x, gsize = gridDim.x * gridDim.y;
            if (et == 0) q_gmax[gid] = __float_as_uint(fmaxf(fmaxf(smax[0], smax[1]), fmaxf(smax[2], smax[3])));
            for (uint32_t j = gsize + gid * 256u + et; j < fill_to; j += gsize * 256u) q_gmax[j] = 0u;
            return;
        }
    }
    // staging: a thread fetches two blocks of 16 of x per step (32 contiguous bytes each; 16 threads cover the 512
    // bytes of a row) and 4 RT 16-byte chunks of v (a wave covers two rows x 512 contiguous bytes per load).
    // It keeps two whole steps in registers while the one before them is multiplied: that is what keeps bytes in flight.
    uint4 rx[2][4], rv[2][RT * 4];
    auto fetch = [&](uint4 (&qx)[4], uint4 (&qv)[RT * 4], int k0) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int id = i * 256 + tid, row = id >> 4, k = k0 + (id & 15) * 16;
            const uint4* src = reinterpret_cast<const uint4*>(x + (int64_t)min(m0 + row, M - 1) * ldx + k);
            qx[2 * i] = k < K ? src[0] : make_uint4(0u, 0u, 0u, 0u);
            qx[2 * i + 1] = k < K ? src[1] : make_uint4(0u, 0u, 0u, 0u);
        }
#pragma unroll
        for (int i = 0; i < RT * 4; ++i) {
            const int id = i * 256 + tid, row = id >> 5, k = k0 + (id & 31) * 8;
            qv[i] = k < K ? *reinterpret_cast<const uint4*>(v + (int64_t)row * K + k) : make_uint4(0u, 0u, 0u, 0u);
        }
    };
    float gmax = 0.0f;
    uint4 px[(QMODE >= 0 && !EW) ? 4 : 1];
    auto stage = [&](const uint4 (&qx)[4], const uint4 (&qv)[RT * 4]) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int id = i * 256 + tid, row = id >> 4, blk = id & 15;
            *reinterpret_cast<uint4*>(tile + row * NT_STRIDE + blk * 16) = qx[2 * i];
            *reinterpret_cast<uint4*>(tile + row * NT_STRIDE + blk * 16 + 8) = qx[2 * i + 1];
        }
        if constexpr (QMODE >= 0 && !EW) {
#pragma unroll
            for (int i = 0; i < 4; ++i) px[i] = qx[i];
        }
#pragma unroll
        for (int i = 0; i < RT * 4; ++i) {
            const int id = i * 256 + tid;
            *reinterpret_cast<uint4*>(tile + (32 + (id >> 5)) * NT_STRIDE + (id & 31) * 8) = qv[i];
        }
    };
    auto encode = [&](int k0) {
        if constexpr (QMODE >= 0 && !EW) {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int id = i * 256 + tid, row = id >> 4, k = k0 + (id & 15) * 16;
                if (m0 + row < M && k < K) {
                    float val[kBlock];
                    const float none[kBlock] = {};
                    unpack16(px[2 * i], px[2 * i + 1], val);
                    const float am = block_amax(val);
                    gmax = fmaxf(gmax, am);
                    const int64_t ib = (int64_t)(m0 + row) * (K / kBlock) + k / kBlock;
                    q_amax[ib] = (uint16_t)(__float_as_uint(am) >> 16);
                    codes[ib] = encode_block<QMODE < 0 ? 0 : QMODE, false>(val, block_scalar<QMODE < 0 ? 0 : QMODE>(am), none);
                }
            }
        }
    };
    float16_t acc[RT];
#pragma unroll
    for (int j = 0; j < RT; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[j][e] = 0.0f;

    // wave w multiplies the quarter [64 w, 64 w + 64) of every step
    const int foff = (lane & 31) * NT_STRIDE + wave * 64 + (lane >> 5) * 8;
    auto multiply = [&]() {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const bf16x8_t fa = *reinterpret_cast<const bf16x8_t*>(tile + foff + ks * 16);
#pragma unroll
            for (int j = 0; j < RT; ++j) {
                const bf16x8_t fb = *reinterpret_cast<const bf16x8_t*>(tile + (32 + j * 32) * NT_STRIDE + foff + ks * 16);
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb, fa, acc[j], 0, 0, 0);
            }
        }
    };
    // two steps are in flight while a third is multiplied: the time of one step is then half the memory latency
    if (steps > 0) fetch(rx[0], rv[0], kof(0));
    if (steps > 1) fetch(rx[1], rv[1], kof(1));
    for (int st = 0; st < steps; st += 2) {
        stage(rx[0], rv[0]);
        __syncthreads();
        if (st + 2 < steps) fetch(rx[0], rv[0], kof(st + 2));
        multiply();
        encode(kof(st));
        __syncthreads();
        if (st + 1 < steps) {
            stage(rx[1], rv[1]);
            __syncthreads();
            if (st + 3 < steps) fetch(rx[1], rv[1], kof(st + 3));
            multiply();
            encode(kof(st + 1));
            __syncthreads();
        }
    }
    if constexpr (QMODE >= 0 && !EW) {
        const float wm = wave_max(gmax);
        if (lane == 0) smax[wave] = wm;
        __syncthreads();
        const uint32_t gid = blockIdx.y * gridDim.x + blockIdx.x, gsize = gridDim.x * gridDim.y;
        if (tid == 0) q_gmax[gid] = __float_as_uint(fmaxf(fmaxf(smax[0], smax[1]), fmaxf(smax[2], smax[3])));
        for (uint32_t j = gsize + gid * 256u + tid; j < fill_to; j += gsize * 256u) q_gmax[j] = 0u;
    }
    // acc[j][e] of lane l: row m0 + l % 32, column 32 j + 8 (e / 4) + 4 (l / 32) + e % 4.  The four waves hold the four
    // quarters of every step of K: their sums meet in LDS (the staged tile is dead after the last barrier), and
    // wave w finishes the quarter e / 4 == w of the columns, adding the waves' shares in the order 0, 1, 2, 3.
#pragma unroll
    for (int j = 0; j < RT; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) red[((wave * RT + j) * 16 + e) * 64 + lane] = acc[j][e];
    __syncthreads();
    const int m = m0 + (lane & 31);
    if (m >= M) return;
#pragma unroll
    for (int j = 0; j < RT; ++j) {
        const int col = j * 32 + 8 * wave + 4 * (lane >> 5);
        float sum4[4];
        uint32_t h[4], ts[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int ee = 4 * wave + e;
            float sum = red[((0 * RT + j) * 16 + ee) * 64 + lane];
#pragma unroll
            for (int w = 1; w < 4; ++w) sum += red[((w * RT + j) * 16 + ee) * 64 + lane];
            sum4[e] = sum;
        }
        if (part) {                                             // one of several slices: the finishing kernel rounds
            *reinterpret_cast<float4*>(part + ((int64_t)blockIdx.y * M + m) * R + col) = make_float4(sum4[0], sum4[1], sum4[2], sum4[3]);
            continue;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            h[e] = bf16_bits(sum4[e]);
            if (t) ts[e] = bf16_bits(__uint_as_float(h[e] << 16) * bf16_lo(s[col + e]));
        }
        *reinterpret_cast<uint2*>(xv + (int64_t)m * R + col) = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
        if (t) *reinterpret_cast<uint2*>(t + (int64_t)m * R + col) = make_uint2(ts[0] | (ts[1] << 16), ts[2] | (ts[3] << 16));
    }
}

// xv = bf16(sum over slices, ascending), t = bf16(xv * s): four columns per thread
__global__ __launch_bounds__(256) void lowrank_nt_finish_kernel(const float* __restrict__ part, int slices, int64_t MR, int R,
                                                                const uint16_t* __restrict__ s, uint16_t* __restrict__ xv,
                                                                uint16_t* __restrict__ t)
{
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= MR) return;
    float4 a = *reinterpret_cast<const float4*>(part + i);
    for (int k = 1; k < slices; ++k) {
        const float4 b = *reinterpret_cast<const float4*>(part + (int64_t)k * MR + i);
        a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
    }
    const uint32_t h[4] = {bf16_bits(a.x), bf16_bits(a.y), bf16_bits(a.z), bf16_bits(a.w)};
    *reinterpret_cast<uint2*>(xv + i) = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
    if (t) {
        const int col = (int)(i % R);
        uint32_t ts[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) ts[e] = bf16_bits(__uint_as_float(h[e] << 16) * bf16_lo(s[col + e]));
        *reinterpret_cast<uint2*>(t + i) = make_uint2(ts[0] | (ts[1] << 16), ts[2] | (ts[3] << 16));
    }
}

// K slices for M rows: none when the row tiles alone give every compute unit a workgroup (measured: slices then cost
// what the second launch costs); otherwise about two workgroups per compute unit, at least four steps per slice, and
// never more workgroups than the quantizer's partial maxima have room for.
static int nt_slices(int64_t M, int64_t K, size_t workspace_bytes, int64_t R)
{
    const int64_t tiles = (M + 31) / 32, steps = (K + NT_STEP - 1) / NT_STEP, cus = device_cus();
    if (tiles >= cus) return 1;
    int64_t sl = (2 * cus + tiles - 1) / tiles;
    if (sl > steps / 4) sl = steps / 4;
    if (sl * tiles > (int64_t)kDeferredPartials) sl = (int64_t)kDeferredPartials / tiles;
    if (sl > 16) sl = 16;
    while (sl > 1 && (size_t)(sl * M * R * 4) > workspace_bytes) --sl;
    return sl < 1 ? 1 : (int)sl;
}

size_t lowrank_nt_workspace_bytes(int64_t M, int64_t R, int64_t K)
{
    if (M <= 0 || R <= 0 || K <= 0) return 0;
    const int sl = nt_slices(M, K, (size_t)-1, R);
    return sl > 1 ? (size_t)sl * M * R * 4 : 0;
}

// qmode < 0: the product alone.  qmode = METIS_MODE_P32 / _PB16: x (contiguous rows, ldx == K) is quantized on the way,
// codes and the deferred data (partial maxima, parked block maxima) as quantize_row_deferred leaves them.
int lowrank_nt(const void* x, int64_t ldx, const void* v, int64_t M, int64_t R, int64_t K, const void* s, void* xv, void* t,
               hipStream_t st, void* workspace, size_t workspace_bytes, int qmode, void* codes, void* deferred, size_t deferred_size)
{
    if (M < 0 || R <= 0 || K <= 0 || ldx < K) return METIS_E_ARG;
    if ((R != 32 && R != 64 && R != 128) || K % 64 || ldx % 8) return METIS_E_SHAPE;
    if (M == 0) return METIS_OK;
    if (M > INT32_MAX - 32 || K > INT32_MAX) return METIS_E_ARG;
    if (!x || !v || !xv || (t && !s)) return METIS_E_ARG;
    if (((uintptr_t)x % 16) || ((uintptr_t)v % 16) || ((uintptr_t)xv % 8) || ((uintptr_t)t % 8) || ((uintptr_t)s % 2)) return METIS_E_ARG;
    if (workspace && ((uintptr_t)workspace % 16)) return METIS_E_WORKSPACE;
    Workspace q = {nullptr, nullptr, nullptr};
    if (qmode >= 0) {
        if (qmode != METIS_MODE_P32 && qmode != METIS_MODE_PB16) return METIS_E_ARG;
        if (R == 128) return METIS_E_SHAPE;
        if (ldx != K || !codes || ((uintptr_t)codes % 8)) return METIS_E_ARG;
        if ((M + 31) / 32 > (int64_t)kDeferredPartials) return METIS_E_TOO_LARGE;
        if (M * K / kBlock >= (int64_t)1 << 31) return METIS_E_ARG;
        if (const int rc = carve_deferred(deferred, deferred_size, M, K, &q)) return rc;
    }
    const int slices = workspace ? nt_slices(M, K, workspace_bytes, R) : 1;
    float* part = slices > 1 ? static_cast<float*>(workspace) : nullptr;
    const dim3 grid((unsigned)((M + 31) / 32), (unsigned)slices);
    // encoding waves of their own when a compute unit gets one workgroup anyway
    const bool ew = (int64_t)grid.x * grid.y <= (int64_t)device_cus();
#define METIS_NT(RT, Q) METIS_NT2(RT, Q, false)
#define METIS_NT2(RT, Q, E) hipLaunchKernelGGL((lowrank_nt_kernel<RT, Q, E>), grid, dim3((Q >= 0 && E) ? 512 : 256), 0, st, (const uint16_t*)x, ldx, (const uint16_t*)v, \
                                           (const uint16_t*)s, (uint16_t*)xv, (uint16_t*)t, (int)M, (int)K, part, (uint2*)codes, q.amax, \
                                           q.gmax, (uint32_t)kDeferredPartials, measure_int("METIS_NT_ROT", 5))
#define METIS_NTQ(RT) do { if (qmode < 0) METIS_NT(RT, -1); else if (qmode == 0) { if (ew) METIS_NT2(RT, 0, true); else METIS_NT(RT, 0); } \
                           else { if (ew) METIS_NT2(RT, 1, true); else METIS_NT(RT, 1); } } while (0)
    if (R == 32) METIS_NTQ(1);
    else if (R == 64) METIS_NTQ(2);
    else METIS_NT(4, -1);                                      // R = 128 fills the register file with the product alone
#undef METIS_NTQ
#undef METIS_NT2
#undef METIS_NT
    if (hipGetLastError() != hipSuccess) return METIS_E_LAUNCH;
    if (slices > 1) {
        const int64_t MR = M * R;
        hipLaunchKernelGGL(lowrank_nt_finish_kernel, dim3((unsigned)((MR / 4 + 255) / 256)), dim3(256), 0, st, part, slices, MR, (int)R,
                           (const uint16_t*)s, (uint16_t*)xv, (uint16_t*)t);
        if (hipGetLastError() != hipSuccess) return METIS_E_LAUNCH;
    }
    return METIS_OK;
}

// ---------------------------------------------------------------------------------------------
// out[C, R] = sum_l a[l, C] b[l, R]
// ---------------------------------------------------------------------------------------------
template <int RT>
__global__ __launch_bounds__(256) void lowrank_tn_kernel(const uint16_t* __restrict__ a, int64_t lda, const uint16_t* __restrict__ b,
                                                         int L, int C, int steps_per_slice, float* __restrict__ part)
{
    constexpr int R = RT * 32;
    // Staged as loaded, token by token, in slabs of 32 columns: [slab][token][32], 64 bytes per token and slab.  The MFMA
    // fragments (8 consecutive tokens of one column) come out of LDS through the transposing read of gfx950
    // (ds_read_b64_tr_b16: the sixteen lanes of a group hand in sixteen addresses of 4 halves each and lane l receives
    // element l % 4 of the pieces of lanes l / 4, l / 4 + 4, l / 4 + 8, l / 4 + 12 -- established with a probe on the
    // device.  With lane i handing in the piece (token i / 4, columns 4 (i % 4) ..), lane l gets column l of four
    // consecutive tokens), so nothing is scattered element by element.  Rows of 64 bytes keep both the 16-byte writes and the
    // transposing reads free of bank conflicts (rows r .. r + 3 and the two 32-byte halves of a row fall on different banks).
    __shared__ __attribute__((aligned(16))) uint16_t at[2][64 * 32];          // [column slab][token][column]
    __shared__ __attribute__((aligned(16))) uint16_t bt[RT][64 * 32];         // [r slab][token][r]
    __shared__ __attribute__((aligned(16))) float red[2][RT][16][64];         // the two waves that take the second half of each step
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c0 = blockIdx.x * 64, slice = blockIdx.y;
    const int steps_all = (L + 63) / 64;
    const int s0 = slice * steps_per_slice, s1 = min(s0 + steps_per_slice, steps_all);
    // loading: thread -> token tid / 8 (+ 32), 16-byte chunk tid % 8 of the 64 columns; for b, R / 8 chunks per token
    const int lrow = tid >> 3, lch = tid & 7;
    const bool col_live = c0 + lch * 8 < C;                     // C % 8 == 0: a chunk is inside or outside
    constexpr int BCH = R / 8;                                  // 16-byte chunks per token of b: 4, 8 or 16
    constexpr int BPT = 64 * BCH / 256;                         // b chunks per thread: 1, 2 or 4
    uint4 ra[2][2], rbv[2][BPT];
    auto fetch = [&](uint4 (&ra)[2], uint4 (&rbv)[BPT], int st) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int l = st * 64 + i * 32 + lrow;
            ra[i] = (l < L && col_live) ? *reinterpret_cast<const uint4*>(a + (int64_t)l * lda + c0 + lch * 8) : make_uint4(0u, 0u, 0u, 0u);
        }
#pragma unroll
        for (int i = 0; i < BPT; ++i) {
            const int id = i * 256 + tid, l = st * 64 + id / BCH, ch = id % BCH;
            rbv[i] = l < L ? *reinterpret_cast<const uint4*>(b + (int64_t)l * R + ch * 8) : make_uint4(0u, 0u, 0u, 0u);
        }
    };
    auto stage = [&](const uint4 (&ra)[2], const uint4 (&rbv)[BPT]) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
            *reinterpret_cast<uint4*>(&at[lch >> 2][(i * 32 + lrow) * 32 + (lch & 3) * 8]) = ra[i];
#pragma unroll
        for (int i = 0; i < BPT; ++i) {
            const int id = i * 256 + tid, tok = id / BCH, ch = id % BCH;
            *reinterpret_cast<uint4*>(&bt[ch >> 2][tok * 32 + (ch & 3) * 8]) = rbv[i];
        }
    };
    float16_t acc[RT];
#pragma unroll
    for (int j = 0; j < RT; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[j][e] = 0.0f;
    // wave -> 32 columns (wave % 2) and the first or second half (wave / 2) of every 64-token step
    const int ct = wave & 1, kh = wave >> 1;
    // lane l of the MFMA holds column l % 32 and the tokens 8 (l / 32) .. + 7 of a 16-token step; in its group of sixteen
    // lanes it hands in the piece (token i / 4, columns 16 (l / 16 % 2) + 4 (i % 4) ..), i = l % 16
    typedef short short4_t __attribute__((ext_vector_type(4)));
    typedef short short8_t __attribute__((ext_vector_type(8)));
    const int piece = ((lane & 15) >> 2) * 32 + ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
    auto fragment = [&](const uint16_t* slab, int tok0) -> bf16x8_t {
        typedef short4_t __attribute__((address_space(3))) * lds_ptr_t;
        const uint16_t* p = slab + tok0 * 32 + piece;
        const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)p);
        const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(p + 4 * 32));
        const short8_t v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        return __builtin_bit_cast(bf16x8_t, v);
    };
    auto multiply = [&]() {
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int tok0 = (kh * 4 + ks * 2 + (lane >> 5)) * 8;
            const bf16x8_t fa = fragment(at[ct], tok0);
#pragma unroll
            for (int j = 0; j < RT; ++j) {
                const bf16x8_t fb = fragment(bt[j], tok0);
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb, fa, acc[j], 0, 0, 0);
            }
        }
    };
    // two steps in flight while a third is multiplied
    if (s0 < s1) fetch(ra[0], rbv[0], s0);
    if (s0 + 1 < s1) fetch(ra[1], rbv[1], s0 + 1);
    for (int st = s0; st < s1; st += 2) {
        stage(ra[0], rbv[0]);
        __syncthreads();
        if (st + 2 < s1) fetch(ra[0], rbv[0], st + 2);
        multiply();
        __syncthreads();
        if (st + 1 < s1) {
            stage(ra[1], rbv[1]);
            __syncthreads();
            if (st + 3 < s1) fetch(ra[1], rbv[1], st + 3);
            multiply();
            __syncthreads();
        }
    }
    // acc[j][e] of lane l: column c0 + 32 ct + l % 32, r = 32 j + 8 (e / 4) + 4 (l / 32) + e % 4; halves of the steps add up
    if (kh == 1) {
#pragma unroll
        for (int j = 0; j < RT; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) red[ct][j][e][lane] = acc[j][e];
    }
    __syncthreads();
    if (kh == 1) return;
    const int c = c0 + ct * 32 + (lane & 31);
    if (c >= C) return;
    float* dst = part + ((int64_t)slice * C + c) * R;
#pragma unroll
    for (int j = 0; j < RT; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float4 o;
            o.x = acc[j][4 * g] + red[ct][j][4 * g][lane];
            o.y = acc[j][4 * g + 1] + red[ct][j][4 * g + 1][lane];
            o.z = acc[j][4 * g + 2] + red[ct][j][4 * g + 2][lane];
            o.w = acc[j][4 * g + 3] + red[ct][j][4 * g + 3][lane];
            *reinterpret_cast<float4*>(dst + j * 32 + 8 * g + 4 * (lane >> 5)) = o;
        }
}

// adds the token slices in order; out [C, R] or, transposed, [R, C]; bf16 or binary32
__global__ __launch_bounds__(256) void lowrank_tn_finish_kernel(const float* __restrict__ part, int slices, int C, int R, void* __restrict__ out,
                                                                int out_f32, int transpose)
{
    const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (id >= (int64_t)C * R) return;
    float sum = part[id];
    for (int z = 1; z < slices; ++z) sum += part[(int64_t)z * C * R + id];
    const int c = (int)(id / R), r = (int)(id % R);
    const int64_t o = transpose ? (int64_t)r * C + c : id;
    if (out_f32) static_cast<float*>(out)[o] = sum;
    else static_cast<uint16_t*>(out)[o] = (uint16_t)bf16_bits(sum);
}

static int tn_slices(int64_t L, int64_t C, int* steps_per_slice)
{
    const int64_t steps = (L + 63) / 64, groups = (C + 63) / 64;
    int64_t want = (4 * (int64_t)device_cus() + groups - 1) / groups;       // four workgroups per compute unit
    if (want > steps / 4) want = steps / 4;                                 // at least four steps per slice
    if (want < 1) want = 1;
    const int64_t per = (steps + want - 1) / want;
    *steps_per_slice = (int)per;
    return (int)((steps + per - 1) / per);
}

size_t lowrank_tn_workspace_bytes(int64_t L, int64_t C, int64_t R)
{
    if (L <= 0 || C <= 0 || R <= 0) return 0;
    int per;
    return (size_t)tn_slices(L, C, &per) * (size_t)C * (size_t)R * sizeof(float);
}

int lowrank_tn(const void* a, int64_t lda, const void* b, int64_t L, int64_t C, int64_t R, void* out, int out_dtype, int transpose,
               void* workspace, size_t workspace_bytes, hipStream_t st)
{
    if (L < 0 || C <= 0 || R <= 0 || lda < C) return METIS_E_ARG;
    if (out_dtype != METIS_DTYPE_BF16 && out_dtype != METIS_DTYPE_F32) return METIS_E_ARG;
    if ((R != 32 && R != 64 && R != 128) || C % 8 || lda % 8) return METIS_E_SHAPE;
    if (L > INT32_MAX - 64 || C > INT32_MAX - 64) return METIS_E_ARG;
    if (!a || !b || !out) return METIS_E_ARG;
    if (((uintptr_t)a % 16) || ((uintptr_t)b % 16) || ((uintptr_t)out % 4)) return METIS_E_ARG;
    if (!workspace || ((uintptr_t)workspace % 16) || workspace_bytes < lowrank_tn_workspace_bytes(L, C, R)) return METIS_E_WORKSPACE;
    int per;
    const int slices = tn_slices(L, C, &per);
    const dim3 grid((unsigned)((C + 63) / 64), (unsigned)slices);
#define METIS_TN(RT) hipLaunchKernelGGL((lowrank_tn_kernel<RT>), grid, dim3(256), 0, st, (const uint16_t*)a, lda, (const uint16_t*)b, (int)L, \
                                        (int)C, per, (float*)workspace)
    if (R == 32) METIS_TN(1);
    else if (R == 64) METIS_TN(2);
    else METIS_TN(4);
#undef METIS_TN
    if (hipGetLastError() != hipSuccess) return METIS_E_LAUNCH;
    const int64_t n = C * R;
    hipLaunchKernelGGL(lowrank_tn_finish_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, (const float*)workspace, slices, (int)C,
                       (int)R, out, out_dtype == METIS_DTYPE_F32, transpose);
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

}  // namespace metis
