// NVFP4 quantizer kernels for gfx950: block-16 absmax -> E2M1 codes + E4M3 block scales + a
// binary32 tensor scale, round-to-nearest or stochastic rounding, row- or column-blocked.
//
// Replaces the eager op chain of src/Metis/Metis/quant.py:6-36 (RNE) and 273-308 + 137-147
// (stochastic rounding).  HBM-bound integer/byte work: one coalesced read of the bf16 input,
// 0.5 B/element of codes and 1/16 B/element of scales written.
//
// Two-phase structure forced by the arithmetic: the codes depend only on the block's own raw
// scalar (quant.py:27), the scale bytes on the tensor-wide maximum (quant.py:21-23).  Phase 1
// writes codes, parks each block's maximum (2 B per block as bf16; 4 B as binary32 for data that is not
// bf16-valued) and publishes one partial maximum per workgroup; phase 2 turns the parked maxima into E4M3 bytes.
#include "metis_device.h"
#include "metis_host.h"
#include "nvfp4_encode.h"
#include "lowrank_small_steps.h"
#include <atomic>
#include <stdio.h>
#include <stdlib.h>
#include <type_traits>

namespace metis {

// ---------------------------------------------------------------------------------------------
// Phase 1, row-blocked: codes + parked block maxima + per-workgroup maximum.  One block of 16 per
// thread per iteration: thread i <-> block i (32 contiguous bytes, two 16-byte loads).
// ---------------------------------------------------------------------------------------------
// WIDE (binary32 arithmetic only): the values to encode are binary32 values that need not be bf16 values,
// because the input tensor is binary32 (in_f32) and/or a binary32 centre is subtracted first.  The short cuts
// of the bf16 path (div6, the block-level guards of the hardware conversion) are proven for bf16 values only, so
// these instantiations take the block scalar by IEEE division, test every quotient before trusting the hardware
// conversion (encode_rne_wide), and park the block maxima as binary32.
//
// center (optional): one value per column, subtracted before anything else: x - center rounded to the
// arithmetic's dtype, the centred residual of the reference's mean mode (src/Metis/Metis/bitlinear.py:
// 330-333).  binary32 [cols] in binary32 arithmetic (always WIDE then), bf16 [cols] in bf16 arithmetic.
__device__ __forceinline__ float block_scalar_ieee(float amax) { return amax / 6.0f + 1e-9f; }

// Round-to-nearest rows of a contiguous bf16 tensor, the shape every activation and weight has: a kernel of its own
// so that its loop carries no row/column arithmetic at all.  Software-pipelined: the next DEPTH blocks' bytes are in
// flight while the current block is encoded.  Binary32 arithmetic takes the two-operation quotient for every block
// maximum the staged table clears (nvfp4_encode.h).
typedef uint32_t metis_u32x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t metis_u32x4_t __attribute__((ext_vector_type(4)));
template <int MODE> __device__ __forceinline__ uint2 encode_row_block(const float (&v)[kBlock], float am, const uint32_t* table)
{
    if constexpr (MODE == 0) {
        uint32_t w[2];
        encode_rne_p32_tbl<kBlock>(v, am, block_scalar<0>(am), table, w);
        return make_uint2(w[0], w[1]);
    } else {
        return encode_rne_pb16(v, block_scalar<1>(am));
    }
}

// (workgroup `block` of `grid`: a launch may give other blocks to other work)
template <int MODE, int DEPTH>
__device__ __forceinline__ void quant_codes_contig_block(uint32_t block, uint32_t grid, const uint4* __restrict__ x,
                                                         uint2* __restrict__ codes, uint16_t* __restrict__ ws_amax,
                                                         uint32_t* __restrict__ ws_gmax, uint32_t nblocks, uint32_t fill_to)
{
    __shared__ uint32_t table[MODE == 0 ? kQuotientTableWords : 4];
    float gmax = 0.0f;
    const uint32_t step = grid * 256u;
    uint32_t i = block * 256u + threadIdx.x;
    uint4 c0[DEPTH], c1[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
        const uint32_t j = i + d * step;
        c0[d] = c1[d] = make_uint4(0u, 0u, 0u, 0u);
        if (j < nblocks) { c0[d] = x[2 * (size_t)j]; c1[d] = x[2 * (size_t)j + 1]; }
    }
    if constexpr (MODE == 0) stage_quotient_table(table);
    while (i < nblocks) {
        const uint4 a0 = c0[0], a1 = c1[0];
#pragma unroll
        for (int d = 0; d + 1 < DEPTH; ++d) { c0[d] = c0[d + 1]; c1[d] = c1[d + 1]; }
        const uint32_t nxt = i + DEPTH * step;
        if (nxt < nblocks) { c0[DEPTH - 1] = x[2 * (size_t)nxt]; c1[DEPTH - 1] = x[2 * (size_t)nxt + 1]; }
        float v[kBlock];
        unpack16(a0, a1, v);
        const float am = block_amax(v);
        gmax = fmaxf(gmax, am);
        ws_amax[i] = (uint16_t)(__float_as_uint(am) >> 16);        // read again soon by whoever forms the scale bytes
        const uint2 cw = encode_row_block<MODE>(v, am, table);
        __builtin_nontemporal_store((metis_u32x2_t){cw.x, cw.y}, reinterpret_cast<metis_u32x2_t*>(codes) + i);
        i += step;
    }
    publish_group_max(gmax, ws_gmax, fill_to, block, grid);
}

template <int MODE, int DEPTH = 1>
__global__ __launch_bounds__(256) void quant_codes_contig_kernel(const uint4* __restrict__ x, uint2* __restrict__ codes,
                                                                 uint16_t* __restrict__ ws_amax, uint32_t* __restrict__ ws_gmax,
                                                                 uint32_t nblocks, uint32_t fill_to)
{
    quant_codes_contig_block<MODE, DEPTH>(blockIdx.x, gridDim.x, x, codes, ws_amax, ws_gmax, nblocks, fill_to);
}

// A decode-sized activation's quantizer (scale bytes deferred) and the first step of its rank-r projection
// (lowrank_small_steps.h) in one launch: both only read x.  Blocks 0 .. qgrid-1 quantize, the others take one K chunk of
// 64 rows each (R <= 128: four waves cover the columns).
template <int MODE>
__global__ __launch_bounds__(256) void decode_quant_partial_kernel(uint32_t qgrid, const uint4* __restrict__ x, uint2* __restrict__ codes,
                                                                   uint16_t* __restrict__ ws_amax, uint32_t* __restrict__ ws_gmax,
                                                                   uint32_t nblocks, uint32_t fill_to, int64_t ldx,
                                                                   const uint16_t* __restrict__ v, int M, int R, int K, int kc, int chunks,
                                                                   float* __restrict__ lr_ws)
{
    if (blockIdx.x < qgrid) {
        quant_codes_contig_block<MODE, 1>(blockIdx.x, qgrid, x, codes, ws_amax, ws_gmax, nblocks, fill_to);
        return;
    }
    const int b = (int)(blockIdx.x - qgrid);
    lowrank_small_partial_block(b % chunks, b / chunks, reinterpret_cast<const uint16_t*>(x), ldx, v, M, R, K, kc, lr_ws);
}

// The same loop with a centre subtracted first (mean mode, src/Metis/Metis/bitlinear.py:311-336: the tensor that is
// quantized is x - me with the column mean me): contiguous bf16 rows of at most 4096 columns, the centre staged once per
// workgroup in LDS (binary32 [cols] in binary32 arithmetic, bf16 values widened in bf16 arithmetic).  In binary32 arithmetic
// the residuals are binary32 values that need not be bf16 values: the per-quotient encoder and binary32 block maxima, as
// quant_codes_kernel<0, false, true>; in bf16 arithmetic the residual is rounded to bf16 and encoded as any bf16 block.
// A block's column position advances by a fixed amount modulo the row length: no division in the loop.
constexpr int kCentreMaxCols = 4096;
template <int MODE>
__global__ __launch_bounds__(256) void quant_codes_contig_centered_kernel(const uint4* __restrict__ x, const void* __restrict__ center,
                                                                          uint2* __restrict__ codes, void* __restrict__ ws_amax_v,
                                                                          uint32_t* __restrict__ ws_gmax, uint32_t nblocks,
                                                                          uint32_t nbpr, uint32_t fill_to)
{
    // quarter q of block b at cen[q][b]: the 16-byte reads of consecutive lanes (consecutive blocks) are consecutive in LDS
    // (block after block, a lane's four reads would be 64 bytes apart from its neighbour's: four lanes per bank)
    __shared__ float4 cen[4][kCentreMaxCols / kBlock];
    for (uint32_t c = threadIdx.x; c < nbpr * kBlock; c += 256u)
        reinterpret_cast<float*>(&cen[(c % kBlock) / 4u][c / kBlock])[c % 4u] =
            MODE == 0 ? static_cast<const float*>(center)[c] : bf16_lo(static_cast<const uint16_t*>(center)[c]);
    __syncthreads();
    float gmax = 0.0f;
    const uint32_t step = gridDim.x * 256u, step_mod = step % nbpr;
    uint32_t i = blockIdx.x * 256u + threadIdx.x;
    uint32_t cb = i % nbpr;
    uint4 c0 = make_uint4(0u, 0u, 0u, 0u), c1 = c0;
    if (i < nblocks) { c0 = x[2 * (size_t)i]; c1 = x[2 * (size_t)i + 1]; }
    while (i < nblocks) {
        const uint4 a0 = c0, a1 = c1;
        const uint32_t nxt = i + step;
        if (nxt < nblocks) { c0 = x[2 * (size_t)nxt]; c1 = x[2 * (size_t)nxt + 1]; }
        float v[kBlock];
        unpack16(a0, a1, v);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float4 f = cen[q][cb];
            if constexpr (MODE == 0) {
                v[4 * q] -= f.x; v[4 * q + 1] -= f.y; v[4 * q + 2] -= f.z; v[4 * q + 3] -= f.w;
            } else {
                v[4 * q] = rb(v[4 * q] - f.x); v[4 * q + 1] = rb(v[4 * q + 1] - f.y);
                v[4 * q + 2] = rb(v[4 * q + 2] - f.z); v[4 * q + 3] = rb(v[4 * q + 3] - f.w);
            }
        }
        const float am = block_amax(v);
        gmax = fmaxf(gmax, am);
        uint2 cw;
        if constexpr (MODE == 0) {
            static_cast<float*>(ws_amax_v)[i] = am;
            cw = encode_rne_wide(v, block_scalar_ieee(am));
        } else {
            static_cast<uint16_t*>(ws_amax_v)[i] = (uint16_t)(__float_as_uint(am) >> 16);
            cw = encode_rne_pb16(v, block_scalar<1>(am));
        }
        __builtin_nontemporal_store((metis_u32x2_t){cw.x, cw.y}, reinterpret_cast<metis_u32x2_t*>(codes) + i);
        i = nxt;
        cb += step_mod;
        cb = cb >= nbpr ? cb - nbpr : cb;
    }
    publish_group_max(gmax, ws_gmax, fill_to);
}

// HAD: every block is rotated first (NV recipe, hadamard16_forward): the rotated tensor is what gets quantized, as in
// `_quantize_wgrad_operand` and `_get_quantized_weight` of src/Metis/Metis/bitlinear.py:395-405, 577-585.  In bf16
// arithmetic the rotated values are rounded to bf16 (the reference's rotation returns the input dtype); in binary32
// arithmetic they are binary32 values that need not be bf16 values, hence WIDE.
template <int MODE, bool SR, bool WIDE = false, bool HAD = false>
__global__ __launch_bounds__(256) void quant_codes_kernel(
    const void* __restrict__ xv, uint32_t rows, uint32_t cols, int64_t ld, const void* __restrict__ noise,
    uint64_t seed, uint64_t offset, uint2* __restrict__ codes, void* __restrict__ ws_amax_v,
    uint32_t* __restrict__ ws_gmax, uint32_t nblocks, int in_f32, const void* __restrict__ center, uint32_t sign_mask,
    uint32_t fill_to)
{
    static_assert(!WIDE || MODE == 0, "binary32 values imply binary32 arithmetic");
    static_assert(!HAD || WIDE || MODE == 1, "rotated binary32 values are not bf16 values");
    const uint16_t* __restrict__ x = static_cast<const uint16_t*>(xv);
    uint16_t* __restrict__ ws_amax = static_cast<uint16_t*>(ws_amax_v);
    float gmax = 0.0f;
    const uint32_t nbpr = cols / kBlock;      // row layout: blocks per row
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < nblocks; i += gridDim.x * 256u) {
        float v[kBlock], u[kBlock] = {};
        const uint32_t row = i / nbpr, cb = i - row * nbpr;
        if (WIDE && in_f32) {
            const float4* p = reinterpret_cast<const float4*>(static_cast<const float*>(xv) + (int64_t)row * ld + (int64_t)cb * kBlock);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const float4 f = p[c];
                v[4 * c] = f.x; v[4 * c + 1] = f.y; v[4 * c + 2] = f.z; v[4 * c + 3] = f.w;
            }
        } else {
            const uint4* p = reinterpret_cast<const uint4*>(x + (int64_t)row * ld + (int64_t)cb * kBlock);
            unpack16(p[0], p[1], v);
        }
        if (center) {
            if constexpr (MODE == 0) {
                const float4* cp = reinterpret_cast<const float4*>(static_cast<const float*>(center) + (size_t)cb * kBlock);
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const float4 f = cp[c];
                    v[4 * c] -= f.x; v[4 * c + 1] -= f.y; v[4 * c + 2] -= f.z; v[4 * c + 3] -= f.w;
                }
            } else {
                const uint4* cp = reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(center) + (size_t)cb * kBlock);
                float cv[kBlock];
                unpack16(cp[0], cp[1], cv);
#pragma unroll
                for (int j = 0; j < kBlock; ++j) v[j] = rb(v[j] - cv[j]);
            }
        }
        if constexpr (HAD) {
            hadamard16_forward(v, sign_mask);
            if constexpr (MODE == 1) {
#pragma unroll
                for (int j = 0; j < kBlock; ++j) v[j] = rb(v[j]);
            }
        }
        if (SR && noise) {
#pragma unroll
            for (int j = 0; j < kBlock; ++j) {
                int64_t e = (int64_t)i * kBlock + j;
                u[j] = MODE ? bf16_lo(((const uint16_t*)noise)[e]) : ((const float*)noise)[e];
            }
        }
        const float am = block_amax(v);
        gmax = fmaxf(gmax, am);
        if constexpr (WIDE) {
            static_cast<float*>(ws_amax_v)[i] = am;
            const float sc = block_scalar_ieee(am);
            if constexpr (SR) codes[i] = !noise ? encode_sr_hardware<0, true>(v, sc, seed, offset, i) : encode_literal<0, true>(v, sc, u);
            else codes[i] = encode_rne_wide(v, sc);
        } else {
            ws_amax[i] = (uint16_t)(__float_as_uint(am) >> 16);      // am is a bf16 value
            // caller-supplied noise: the reference's literal sequence; own stream: hardware stochastic rounding
            codes[i] = (SR && !noise) ? encode_sr_hardware<MODE>(v, block_scalar<MODE>(am), seed, offset, i)
                                      : encode_block<MODE, SR>(v, block_scalar<MODE>(am), u);
        }
    }
    publish_group_max(gmax, ws_gmax, fill_to);
}

// ---------------------------------------------------------------------------------------------
// Phase 1, column-blocked: blocks run down 16 consecutive rows of one column and the packed tensor
// is stored transposed ([cols, rows/2] codes, [cols, rows/16] scales).  A workgroup owns a tile of
// 256 rows x 64 columns: thread t encodes blocks 4g..4g+3 (g = t / 64) of column t % 64, every load
// instruction reading 64 consecutive columns of one row.  Codes and block maxima are transposed
// through LDS so that they leave as 32-byte (8-byte) pieces of the 128 (32) contiguous bytes each
// column owns in the tile, instead of one scattered 8-byte and 2-byte store per lane.
// ---------------------------------------------------------------------------------------------
constexpr int kColTileBlocks = 16, kColTileCols = 64;
// F32IN (WIDE only): the input tensor itself is binary32; a compile-time choice, so that the sixteen loads of a block are
// issued back to back (decided at run time, element by element, the bf16 input of a centred call took twice as long).
template <int MODE, bool SR, bool WIDE = false, bool F32IN = false>
__global__ __launch_bounds__(256) void quant_codes_col_kernel(
    const void* __restrict__ xv, uint32_t rows, uint32_t cols, int64_t ld, const void* __restrict__ noise,
    uint64_t seed, uint64_t offset, uint2* __restrict__ codes, void* __restrict__ ws_amax_v,
    uint32_t* __restrict__ ws_gmax, uint32_t tiles_c, uint32_t tiles_total, const void* __restrict__ center)
{
    static_assert(!F32IN || WIDE, "binary32 input implies binary32 values");
    static_assert(!WIDE || MODE == 0, "binary32 values imply binary32 arithmetic");
    using amax_t = typename std::conditional<WIDE, float, uint16_t>::type;   // parked block maximum
    const uint16_t* __restrict__ x = static_cast<const uint16_t*>(xv);
    amax_t* __restrict__ ws_amax = static_cast<amax_t*>(ws_amax_v);
    __shared__ uint2 s_codes[kColTileCols][kColTileBlocks + 1];
    __shared__ amax_t s_amax[kColTileCols][kColTileBlocks + 2];
    const uint32_t nbc = rows / kBlock;                       // blocks per column
    const uint32_t cl = threadIdx.x & 63u, g = threadIdx.x >> 6;
    float gmax = 0.0f;
    for (uint32_t tile = blockIdx.x; tile < tiles_total; tile += gridDim.x) {
        const uint32_t tr = tile / tiles_c, tc = tile - tr * tiles_c;
        const uint32_t c = tc * kColTileCols + cl;
#pragma unroll 1
        for (uint32_t k = 0; k < 4u; ++k) {
            const uint32_t bl = g * 4u + k, b = tr * kColTileBlocks + bl;
            uint2 packed = make_uint2(0u, 0u);
            float am = 0.0f;
            if (c < cols && b < nbc) {
                float v[kBlock], u[kBlock] = {};
#pragma unroll
                for (int j = 0; j < kBlock; ++j) {
                    if constexpr (F32IN) v[j] = static_cast<const float*>(xv)[(int64_t)(b * kBlock + j) * ld + c];
                    else v[j] = bf16_lo(x[(int64_t)(b * kBlock + j) * ld + c]);
                }
                if (center) {                                  // one centre per column: the same for the whole block
                    if constexpr (MODE == 0) {
                        const float cen = static_cast<const float*>(center)[c];
#pragma unroll
                        for (int j = 0; j < kBlock; ++j) v[j] -= cen;
                    } else {
                        const float cen = bf16_lo(static_cast<const uint16_t*>(center)[c]);
#pragma unroll
                        for (int j = 0; j < kBlock; ++j) v[j] = rb(v[j] - cen);
                    }
                }
                if (SR && noise) {
#pragma unroll
                    for (int j = 0; j < kBlock; ++j) {
                        int64_t e = (int64_t)(b * kBlock + j) * cols + c;
                        u[j] = MODE ? bf16_lo(((const uint16_t*)noise)[e]) : ((const float*)noise)[e];
                    }
                }
                am = block_amax(v);
                gmax = fmaxf(gmax, am);
                if constexpr (WIDE) {
                    const float sc = block_scalar_ieee(am);
                    if constexpr (SR) packed = !noise ? encode_sr_hardware<0, true>(v, sc, seed, offset, (int64_t)c * nbc + b)
                                                      : encode_literal<0, true>(v, sc, u);
                    else packed = encode_rne_wide(v, sc);
                } else {
                    packed = (SR && !noise) ? encode_sr_hardware<MODE>(v, block_scalar<MODE>(am), seed, offset, (int64_t)c * nbc + b)
                                            : encode_block<MODE, SR>(v, block_scalar<MODE>(am), u);
                }
            }
            s_codes[cl][bl] = packed;
            if constexpr (WIDE) s_amax[cl][bl] = am;
            else s_amax[cl][bl] = (uint16_t)(__float_as_uint(am) >> 16);
        }
        __syncthreads();
        {   // column t / 4, blocks 4 (t % 4) .. +3 of the tile: 32 contiguous bytes of codes, 8 of maxima
            const uint32_t oc = threadIdx.x >> 2, part = threadIdx.x & 3u;
            const uint32_t c2 = tc * kColTileCols + oc, b0 = tr * kColTileBlocks + part * 4u;
            if (c2 < cols) {
#pragma unroll
                for (uint32_t i = 0; i < 4u; ++i) {
                    if (b0 + i < nbc) {
                        const int64_t ob = (int64_t)c2 * nbc + b0 + i;
                        codes[ob] = s_codes[oc][part * 4u + i];
                        ws_amax[ob] = s_amax[oc][part * 4u + i];
                    }
                }
            }
        }
        __syncthreads();
    }
    publish_group_max(gmax, ws_gmax);
}

// ---------------------------------------------------------------------------------------------
// Phase 1 of BOTH packings of one tensor in one pass: the weight-gradient and input-gradient GEMMs of the backward
// pass contract the output gradient over different dimensions, so dY is packed twice -- blocks along its last
// dimension (rows) and blocks down its columns (src/Metis/Metis/bitlinear.py:488-510 re-quantizes grad_output for
// each product).  Stochastic rounding on the library's own stream; the two packings draw from their own offsets, so the
// results are those of quant_codes_kernel<.., SR> and quant_codes_col_kernel<.., SR> called one after the other.
// Same tile as the column kernel (256 rows x 64 columns per workgroup, wave g takes 16-row slabs 4g .. 4g+3): a lane
// holds one column of a slab; the slab also goes through LDS (68-word rows) and comes back as row blocks, lane l
// taking row l / 4, block l % 4.  Both packings share the tensor maximum, hence one partial maximum per workgroup.
// ---------------------------------------------------------------------------------------------
constexpr uint32_t kBothRun = 16;
template <int MODE, bool WIDE = false>
__global__ __launch_bounds__(256) void quant_codes_both_kernel(
    const void* __restrict__ xv, uint32_t rows, uint32_t cols, int64_t ld, uint64_t seed, uint64_t offset_row, uint64_t offset_col,
    uint2* __restrict__ codes_row, void* __restrict__ amax_row_v, uint2* __restrict__ codes_col, void* __restrict__ amax_col_v,
    uint32_t* __restrict__ ws_gmax, uint32_t tiles_c, uint32_t tiles_total)
{
    static_assert(!WIDE || MODE == 0, "binary32 values imply binary32 arithmetic");
    using amax_t = typename std::conditional<WIDE, float, uint16_t>::type;
    amax_t* __restrict__ amax_row = static_cast<amax_t*>(amax_row_v);
    amax_t* __restrict__ amax_col = static_cast<amax_t*>(amax_col_v);
    __shared__ uint2 s_codes[kColTileCols][kColTileBlocks + 1];
    __shared__ amax_t s_amax[kColTileCols][kColTileBlocks + 2];
    // one 16 x 64 slab per wave, in the input's own width: binary32 words, or bf16 pairs as loaded
    constexpr int kSlabWords = WIDE ? kColTileCols + 4 : kColTileCols / 2 + 4;
    __shared__ __attribute__((aligned(16))) uint32_t slab[4][kBlock][kSlabWords];
    const uint32_t nbc = rows / kBlock, nbpr = cols / kBlock;
    const uint32_t lane = threadIdx.x & 63u, g = threadIdx.x >> 6;
    const uint32_t rr = lane >> 2, cb = lane & 3u;            // as a row block: row rr of the slab, block cb of its 64 columns
    float gmax = 0.0f;
    auto parked = [](float am) -> amax_t {
        if constexpr (WIDE) return am;
        else return (uint16_t)(__float_as_uint(am) >> 16);
    };
    // A tile's row blocks are 32 bytes of a row of codes, and 8 bytes of a row of maxima: kBothRun tiles side by side
    // complete whole 128-byte lines.  Workgroups go round the eight dies in turn, each die with an L2 of its own that
    // merges partial lines; so the workgroups of one die take a run of kBothRun neighbouring tiles at a time.
    const uint32_t span = 8u * kBothRun, padded = (tiles_total + span - 1) / span * span;
    auto tile_of = [&](uint32_t wid) { return wid / span * span + (wid % 8u) * kBothRun + (wid / 8u) % kBothRun; };
    // slab k of workgroup item wid, as the wave loads it: instruction i covers RPI whole rows of the slab, consecutive lanes
    // consecutive 16-byte chunks (every instruction reads whole lines); zeros beyond the tensor.  The next slab's loads are
    // issued before the current one is encoded (one slab ahead, across tiles).
    constexpr int NQ = WIDE ? 4 : 2, CPR = WIDE ? 16 : 8, RPI = 64 / CPR;   // loads per lane, 16-byte chunks per slab row, rows per load
    static_assert(NQ * RPI == kBlock, "the instructions of a wave cover the 16 rows of a slab");
    const uint32_t lrow = lane / CPR, lch = lane % CPR;        // row within an instruction's rows, 16-byte chunk of the row
    auto fetch = [&](uint32_t wid, uint32_t k, uint4 (&q)[NQ]) {
#pragma unroll
        for (int i = 0; i < NQ; ++i) q[i] = make_uint4(0u, 0u, 0u, 0u);
        if (wid >= padded) return;
        const uint32_t tile = tile_of(wid);
        if (tile >= tiles_total) return;
        const uint32_t tr = tile / tiles_c, tc = tile - tr * tiles_c;
        const uint32_t b = tr * kColTileBlocks + g * 4u + k;
        const uint32_t col = tc * kColTileCols + lch * (WIDE ? 4u : 8u);
        if (b < nbc && col < cols) {
#pragma unroll
            for (int i = 0; i < NQ; ++i) {
                const int64_t at = (int64_t)(b * kBlock + i * RPI + lrow) * ld + col;
                q[i] = WIDE ? *reinterpret_cast<const uint4*>(static_cast<const float*>(xv) + at)
                            : *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(xv) + at);
            }
        }
    };
    uint4 cur[NQ], nxt[NQ];
    fetch(blockIdx.x, 0u, cur);
    for (uint32_t wid = blockIdx.x; wid < padded; wid += gridDim.x) {
        const uint32_t tile = tile_of(wid);
        const bool live = tile < tiles_total;                  // the same for the whole workgroup
        const uint32_t tr = tile / tiles_c, tc = tile - tr * tiles_c;
        const uint32_t c = tc * kColTileCols + lane;
        const uint32_t cbg = tc * 4u + cb;
#pragma unroll 1
        for (uint32_t k = 0; k < 4u; ++k) {
            if (k < 3u) fetch(wid, k + 1u, nxt);
            else fetch(wid + gridDim.x, 0u, nxt);
            if (live) {
                const uint32_t bl = g * 4u + k, b = tr * kColTileBlocks + bl;
                // to this wave's slab in LDS as loaded, and back as columns.  A wave's LDS operations complete in the
                // order issued, so no wait lies between its own writes and reads: the barriers only keep the compiler
                // from moving them.
                float w[kBlock], v[kBlock];
                const bool have_row = b < nbc && cbg < nbpr;
#pragma unroll
                for (int i = 0; i < NQ; ++i) *reinterpret_cast<uint4*>(&slab[g][i * RPI + lrow][lch * 4u]) = cur[i];
                __builtin_amdgcn_wave_barrier();
                if constexpr (WIDE) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const uint4 f = *reinterpret_cast<const uint4*>(&slab[g][rr][cb * kBlock + 4 * q]);
                        w[4 * q] = __uint_as_float(f.x); w[4 * q + 1] = __uint_as_float(f.y);
                        w[4 * q + 2] = __uint_as_float(f.z); w[4 * q + 3] = __uint_as_float(f.w);
                    }
#pragma unroll
                    for (int j = 0; j < kBlock; ++j) v[j] = __uint_as_float(slab[g][j][lane]);
                } else {
                    unpack16(*reinterpret_cast<const uint4*>(&slab[g][rr][cb * 8u]), *reinterpret_cast<const uint4*>(&slab[g][rr][cb * 8u + 4u]), w);
                    const uint32_t shift = (lane & 1u) ? 0u : 16u;  // a bf16 is the upper half of its binary32 value
#pragma unroll
                    for (int j = 0; j < kBlock; ++j) v[j] = __uint_as_float((slab[g][j][lane >> 1] << shift) & 0xffff0000u);
                }
                __builtin_amdgcn_wave_barrier();
                if (have_row) {
                    const float amr = block_amax(w);
                    gmax = fmaxf(gmax, amr);
                    const int64_t ir = (int64_t)(b * kBlock + rr) * nbpr + cbg;
                    uint2 pr;
                    if constexpr (WIDE) pr = encode_sr_hardware<0, true>(w, block_scalar_ieee(amr), seed, offset_row, ir);
                    else pr = encode_sr_hardware<MODE>(w, block_scalar<MODE>(amr), seed, offset_row, ir);
                    codes_row[ir] = pr;
                    amax_row[ir] = parked(amr);
                }
                uint2 packed = make_uint2(0u, 0u);
                float am = 0.0f;
                if (c < cols && b < nbc) {
                    am = block_amax(v);
                    if constexpr (WIDE) packed = encode_sr_hardware<0, true>(v, block_scalar_ieee(am), seed, offset_col, (int64_t)c * nbc + b);
                    else packed = encode_sr_hardware<MODE>(v, block_scalar<MODE>(am), seed, offset_col, (int64_t)c * nbc + b);
                }
                s_codes[lane][bl] = packed;
                s_amax[lane][bl] = parked(am);
            }
#pragma unroll
            for (int i = 0; i < NQ; ++i) cur[i] = nxt[i];
        }
        if (!live) continue;
        __syncthreads();
        {   // column t / 4, blocks 4 (t % 4) .. +3 of the tile: 32 contiguous bytes of codes, 8 of maxima
            const uint32_t oc = threadIdx.x >> 2, part = threadIdx.x & 3u;
            const uint32_t c2 = tc * kColTileCols + oc, b0 = tr * kColTileBlocks + part * 4u;
            if (c2 < cols) {
#pragma unroll
                for (uint32_t i = 0; i < 4u; ++i) {
                    if (b0 + i < nbc) {
                        const int64_t ob = (int64_t)c2 * nbc + b0 + i;
                        codes_col[ob] = s_codes[oc][part * 4u + i];
                        amax_col[ob] = s_amax[oc][part * 4u + i];
                    }
                }
            }
        }
        __syncthreads();
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
                                                           uint32_t nblocks, const uint16_t* __restrict__ ws_amax2 = nullptr,
                                                           uint8_t* __restrict__ scales2 = nullptr, float* __restrict__ unit_out2 = nullptr)
{
    // grid row 1 (if launched): a second packing of the same tensor (same partial maxima, its own parked block maxima)
    if (blockIdx.y) { ws_amax = ws_amax2; scales = scales2; unit_out = unit_out2; }
    __shared__ float smax[4];
    const uint32_t nocts = nblocks / 8u;
    const uint32_t step = gridDim.x * 256u;
    uint32_t q = blockIdx.x * 256u + threadIdx.x;
    // first eight parked maxima are requested before the reduction so that both round trips overlap
    uint4 a = make_uint4(0u, 0u, 0u, 0u);
    if (q < nocts) a = reinterpret_cast<const uint4*>(ws_amax)[q];
    float m = 0.0f;
    for (uint32_t g = threadIdx.x; g < ngroups; g += 256u) m = fmaxf(m, __uint_as_float(ws_gmax[g]));
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) smax[threadIdx.x >> 6] = m;
    __syncthreads();
    const float amax = fmaxf(fmaxf(smax[0], smax[1]), fmaxf(smax[2], smax[3]));
    // max over blocks of scalar(amax_block) = scalar(max amax_block): the scalar map is monotone
    const float unit = tensor_unit_of<MODE>(amax);
    if (blockIdx.x == 0 && threadIdx.x == 0) *unit_out = unit;

    auto four_bytes = [&](uint32_t w0, uint32_t w1) {
        const float t0 = rd<MODE>(block_scalar<MODE>(bf16_lo(w0)) / unit);
        const float t1 = rd<MODE>(block_scalar<MODE>(bf16_hi(w0)) / unit);
        const float t2 = rd<MODE>(block_scalar<MODE>(bf16_lo(w1)) / unit);
        const float t3 = rd<MODE>(block_scalar<MODE>(bf16_hi(w1)) / unit);
        const int w = __builtin_amdgcn_cvt_pk_fp8_f32(t0, t1, 0, false);
        return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(t2, t3, w, true);
    };
    while (q < nocts) {
        const uint32_t nxt = q + step;
        uint4 n = a;
        if (nxt < nocts) n = reinterpret_cast<const uint4*>(ws_amax)[nxt];
        uint2 o;
        o.x = four_bytes(a.x, a.y);
        o.y = four_bytes(a.z, a.w);
        reinterpret_cast<uint2*>(scales)[q] = o;
        a = n; q = nxt;
    }
    // ragged tail (block count not a multiple of eight)
    for (uint32_t k = nocts * 8u + blockIdx.x * 256u + threadIdx.x; k < nblocks; k += step) {
        const float s = block_scalar<MODE>(__uint_as_float((uint32_t)ws_amax[k] << 16));
        scales[k] = (uint8_t)e4m3_byte(rd<MODE>(s / unit));
    }
}

// Phase 2 for a decode-sized activation (fewer than 256 rows, cols % 256 == 0): unit and scale bytes as above, and the
// packed tensor once more in the decode layout that the decode-sized GEMM streams as whole lines (gemm_common.h): block
// (tile of 32 rows, step of 256 elements) = four KiB of codes, piece j of lane l = (h << 5 | row) at j * 1024 + l * 16,
// then 512 scale bytes, lane l at 4096 + l * 8.  One workgroup per block at a time: thread (j, l) moves a piece, and the
// threads with j == 0 form the eight scale bytes of their lane.  Rows past the tensor are zero.
template <int MODE>
__global__ __launch_bounds__(256) void quant_scales_decode_kernel(const uint16_t* __restrict__ ws_amax, const uint32_t* __restrict__ ws_gmax,
                                                                  uint32_t ngroups, const uint8_t* __restrict__ codes,
                                                                  uint8_t* __restrict__ scales, float* __restrict__ unit_out,
                                                                  uint8_t* __restrict__ decode, int rows, int cols, int blocks)
{
    __shared__ float smax[4];
    float m = 0.0f;
    for (uint32_t g = threadIdx.x; g < ngroups; g += 256u) m = fmaxf(m, __uint_as_float(ws_gmax[g]));
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) smax[threadIdx.x >> 6] = m;
    __syncthreads();
    const float unit = tensor_unit_of<MODE>(fmaxf(fmaxf(smax[0], smax[1]), fmaxf(smax[2], smax[3])));
    if (blockIdx.x == 0 && threadIdx.x == 0) *unit_out = unit;
    const int iters = cols / 256, l = threadIdx.x & 63, j = threadIdx.x >> 6, h = l >> 5;
    for (int b = blockIdx.x; b < blocks; b += gridDim.x) {
        const int tile = b / iters, it = b - tile * iters;
        const int row = tile * 32 + (l & 31);
        uint8_t* dst = decode + (int64_t)b * kDecodeBlock;
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        if (row < rows) v = *reinterpret_cast<const uint4*>(codes + (int64_t)row * (cols / 2) + it * 128 + h * 64 + 16 * j);
        *reinterpret_cast<uint4*>(dst + j * 1024 + l * 16) = v;
        if (j == 0) {
            uint2 o = make_uint2(0u, 0u);
            if (row < rows) {
                const int64_t kb = (int64_t)row * (cols / kBlock) + it * 16 + h * 8;
                const uint4 a = *reinterpret_cast<const uint4*>(ws_amax + kb);
                uint32_t by[8];
                const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    by[2 * q] = scale_byte_of<MODE>(w[q] & 0xffffu, unit);
                    by[2 * q + 1] = scale_byte_of<MODE>(w[q] >> 16, unit);
                }
                o.x = by[0] | (by[1] << 8) | (by[2] << 16) | (by[3] << 24);
                o.y = by[4] | (by[5] << 8) | (by[6] << 16) | (by[7] << 24);
                *reinterpret_cast<uint2*>(scales + kb) = o;
            }
            *reinterpret_cast<uint2*>(dst + 4096 + l * 8) = o;
        }
    }
}

// Phase 2 for parked binary32 maxima (binary32 input): IEEE divisions, four blocks per thread.
__global__ __launch_bounds__(256) void quant_scales_f32_kernel(const float* __restrict__ ws_amax,
                                                               const uint32_t* __restrict__ ws_gmax, uint32_t ngroups,
                                                               uint8_t* __restrict__ scales, float* __restrict__ unit_out,
                                                               uint32_t nblocks, const float* __restrict__ ws_amax2 = nullptr,
                                                               uint8_t* __restrict__ scales2 = nullptr, float* __restrict__ unit_out2 = nullptr)
{
    if (blockIdx.y) { ws_amax = ws_amax2; scales = scales2; unit_out = unit_out2; }
    __shared__ float smax[4];
    float m = 0.0f;
    for (uint32_t g = threadIdx.x; g < ngroups; g += 256u) m = fmaxf(m, __uint_as_float(ws_gmax[g]));
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) smax[threadIdx.x >> 6] = m;
    __syncthreads();
    const float amax = fmaxf(fmaxf(smax[0], smax[1]), fmaxf(smax[2], smax[3]));
    const float unit = block_scalar_ieee(amax) / 448.0f;      // the scalar map is monotone: max of scalars = scalar of max
    if (blockIdx.x == 0 && threadIdx.x == 0) *unit_out = unit;
    const uint32_t nquads = nblocks / 4u, step = gridDim.x * 256u;
    for (uint32_t q = blockIdx.x * 256u + threadIdx.x; q < nquads; q += step) {
        const float4 a = reinterpret_cast<const float4*>(ws_amax)[q];
        const int w = __builtin_amdgcn_cvt_pk_fp8_f32(block_scalar_ieee(a.x) / unit, block_scalar_ieee(a.y) / unit, 0, false);
        reinterpret_cast<uint32_t*>(scales)[q] =
            (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(block_scalar_ieee(a.z) / unit, block_scalar_ieee(a.w) / unit, w, true);
    }
    for (uint32_t k = nquads * 4u + blockIdx.x * 256u + threadIdx.x; k < nblocks; k += step)
        scales[k] = (uint8_t)e4m3_byte(block_scalar_ieee(ws_amax[k]) / unit);
}

// ---------------------------------------------------------------------------------------------
// Single-launch variant for round-to-nearest rows of a contiguous bf16 tensor: both phases in one kernel.  Each thread
// keeps the maxima of its (at most NB) blocks in registers across a grid-wide maximum, so in the ordinary case neither
// the parked maxima nor a second launch are needed.
//
// The grid-wide maximum does not assume that all workgroups are resident together.  Workgroups arrive through a
// two-level tree (64 groups of up to 64 workgroups) whose nodes are a maximum and an arrival counter, each updated by one
// read-modify-write, so exactly one workgroup learns that it is the LAST to arrive and what the tensor maximum is.  It
// exchanges {call tag, result, maximum} into 64 words (one per group, a line each), writes the tensor unit, and cleans
// the tree for the next call.  Every other workgroup polls its group's word a bounded number of times.  One that gives
// up -- because part of the grid is still waiting for a compute unit, held by another kernel or by these very pollers
// -- parks its block maxima in the workspace, raises its flag, swaps {call tag, "somebody left"} into its group's word
// and exits WITHOUT its scale bytes: the last workgroup finds that marker in what its exchange returns and writes
// those bytes itself.  If the exchange came first, the leaver's swap fails, it reads the result and finishes its own
// bytes after all.  That decision hangs on one word, so relaxed device-scope atomics suffice on the ordinary path (an
// acquire or release at device scope writes back or invalidates a whole L2 on this part); only a workgroup that leaves
// and the last workgroup that cleans up after one pay for fences.  Every wave exits after a bounded time whatever else
// runs on the device, and the result is always complete and always the same bytes as the two-launch path.
// The area starts zero-filled; a call leaves the tree clean and only tagged words behind.
// ---------------------------------------------------------------------------------------------
constexpr uint32_t kSpinLimit = 4096;            // polls (roughly a microsecond each) before a workgroup leaves its scale bytes behind
constexpr uint32_t kGroups = 64;                 // groups, and the most members a group can have
constexpr int kFusedMaxGrid = kGroups * kGroups;
// locations inside the synchronisation area (uint32 units)
__device__ __forceinline__ uint64_t* sync_generation(uint32_t* s) { return reinterpret_cast<uint64_t*>(s); }
__device__ __forceinline__ uint32_t* sync_top(uint32_t* s) { return s + 4; }                           // {maximum, arrivals}
__device__ __forceinline__ uint32_t* sync_group(uint32_t* s, uint32_t j) { return s + 64 + j * 32; }     // {maximum, arrivals}, a line each
__device__ __forceinline__ uint64_t* sync_result(uint32_t* s, uint32_t j) { return reinterpret_cast<uint64_t*>(s + 2176 + j * 32); }
__device__ __forceinline__ uint32_t* sync_left_flag(uint32_t* s, uint32_t b) { return s + 4224 + b; }
static_assert((4224 + kFusedMaxGrid) * 4 <= kWsSyncBytes, "synchronisation area too small");

#define METIS_AT_LOAD(p) __hip_atomic_load((p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define METIS_AT_STORE(p, v) __hip_atomic_store((p), (v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define METIS_AT_CAS(p, expected, desired) \
    __hip_atomic_compare_exchange_strong((p), (expected), (desired), __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define METIS_AT_XCHG(p, v) __hip_atomic_exchange((p), (v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)

// a group's result word: tag << 18 | kind << 16 | bf16 payload; kind 0: the tensor maximum, kind 1: a member has left
__device__ __forceinline__ uint64_t result_word(uint64_t tag, uint32_t kind, uint32_t payload) { return (tag << 18) | ((uint64_t)kind << 16) | payload; }
__device__ __forceinline__ bool is_result(uint64_t w, uint64_t tag) { return (w >> 16) == (tag << 2); }
__device__ __forceinline__ bool is_left_marker(uint64_t w, uint64_t tag) { return (w >> 16) == ((tag << 2) | 1u); }

struct GridMaxState {
    float wave_part[4];
    uint32_t last;               // this workgroup was the last to arrive
    uint32_t known;              // result holds the tensor maximum
    float result;
    uint32_t nleft;
    uint32_t left[256];          // workgroups of one slab of 256 flags that left their scale bytes behind
};

// Every thread, at kernel start (before its workgroup arrives, so before the counter can move): the tag of this call.
__device__ __forceinline__ uint64_t grid_max_begin(uint32_t* sync)
{
    return METIS_AT_LOAD(sync_generation(sync)) + 1u;
}

// One more arrival with maximum `bits` at a tree node {maximum, arrivals}; true for the arrival that completes `expected`,
// with the node's maximum.  Two relaxed read-modify-writes without retry: the counter's increment is made to depend on
// the value the maximum's returns, so it is issued only after the maximum has been performed at the coherence point; the
// arrival that sees the count complete therefore reads a maximum that every earlier arrival has folded in.
__device__ __forceinline__ bool tree_arrive(uint32_t* node, uint32_t bits, uint32_t expected, uint32_t& folded)
{
    const uint32_t before = __hip_atomic_fetch_max(node, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint32_t one = 1u + (before >> 31);                      // bit 31 of a non-negative float's pattern: always 0
    if (__hip_atomic_fetch_add(node + 1, one, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != expected - 1u) return false;
    folded = METIS_AT_LOAD(node);
    METIS_AT_STORE(node, 0u);                                      // nobody else touches the node before the next call
    METIS_AT_STORE(node + 1, 0u);
    return true;
}

// Called by every thread of every workgroup, once: folds the workgroup maximum (a bf16 value) into the tree.
__device__ __forceinline__ void grid_max_arrive(float thread_max, uint32_t* sync, GridMaxState& sh)
{
    const float m = wave_max(thread_max);
    if ((threadIdx.x & 63) == 0) sh.wave_part[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t bits = __float_as_uint(fmaxf(fmaxf(sh.wave_part[0], sh.wave_part[1]), fmaxf(sh.wave_part[2], sh.wave_part[3])));
        const uint32_t j = blockIdx.x % kGroups;
        const uint32_t ngroups = gridDim.x < kGroups ? gridDim.x : kGroups;
        const uint32_t members = (gridDim.x + kGroups - 1u - j) / kGroups;
        uint32_t gm = 0u, fin = 0u;
        const bool last = tree_arrive(sync_group(sync, j), bits, members, gm) && tree_arrive(sync_top(sync), gm, ngroups, fin);
        sh.last = last ? 1u : 0u;
        sh.known = sh.last;
        sh.result = __uint_as_float(fin);
    }
}

// One block in flight ahead of the one being encoded (as in phase 1 of the two-launch path), block maxima kept in
// registers, and the arrival placed before the encoding of the thread's last block so that the tree's latency is covered.
template <int MODE, int NB>
__global__ __launch_bounds__(256) void quant_fused_kernel(const uint16_t* __restrict__ x, uint2* __restrict__ codes,
                                                          uint8_t* __restrict__ scales, float* __restrict__ unit_out,
                                                          uint32_t* __restrict__ sync, uint16_t* __restrict__ parked,
                                                          uint32_t nblocks, uint32_t spin_limit)
{
    __shared__ GridMaxState sh;
    const uint64_t tag = grid_max_begin(sync);
    const uint32_t stride = gridDim.x * 256u;
    const uint32_t i0 = blockIdx.x * 256u + threadIdx.x;
    const uint4* xp = reinterpret_cast<const uint4*>(x);
    uint4 c0 = make_uint4(0u, 0u, 0u, 0u), c1 = c0;
    if (i0 < nblocks) { c0 = xp[2 * (size_t)i0]; c1 = xp[2 * (size_t)i0 + 1]; }
    float am[NB];
    float gmax = 0.0f;
    const float none[kBlock] = {};
    constexpr int TAIL = NB >= 2 ? 2 : 1;                          // blocks encoded after the arrival
#pragma unroll
    for (int k = 0; k < NB - TAIL; ++k) {
        const uint32_t i = i0 + k * stride;
        uint4 n0 = make_uint4(0u, 0u, 0u, 0u), n1 = n0;
        if (i + stride < nblocks) { n0 = xp[2 * (size_t)(i + stride)]; n1 = xp[2 * (size_t)(i + stride) + 1]; }
        float v[kBlock];
        unpack16(c0, c1, v);
        am[k] = block_amax(v);
        gmax = fmaxf(gmax, am[k]);
        if (i < nblocks) codes[i] = encode_block<MODE, false>(v, block_scalar<MODE>(am[k]), none);
        c0 = n0; c1 = n1;
    }
    {
        // the last blocks: all their maxima first, then the arrival, then their encoding -- a few microseconds of vector
        // work between the arrival and the wait, which is what the tree and the last workgroup's word need to get round
        const uint32_t ia = i0 + (NB - TAIL) * stride, ib = ia + stride;
        uint4 d0 = make_uint4(0u, 0u, 0u, 0u), d1 = d0;
        if (TAIL == 2 && ib < nblocks) { d0 = xp[2 * (size_t)ib]; d1 = xp[2 * (size_t)ib + 1]; }
        float va[kBlock], vb[kBlock];
        unpack16(c0, c1, va);
        am[NB - TAIL] = block_amax(va);
        gmax = fmaxf(gmax, am[NB - TAIL]);
        if (TAIL == 2) {
            unpack16(d0, d1, vb);
            am[NB - 1] = block_amax(vb);
            gmax = fmaxf(gmax, am[NB - 1]);
        }
        grid_max_arrive(gmax, sync, sh);
        if (ia < nblocks) codes[ia] = encode_block<MODE, false>(va, block_scalar<MODE>(am[NB - TAIL]), none);
        if (TAIL == 2 && ib < nblocks) codes[ib] = encode_block<MODE, false>(vb, block_scalar<MODE>(am[NB - 1]), none);
    }
    auto scale_bytes = [&](float amax) {
        const float unit = rd<MODE>(block_scalar<MODE>(amax) / 448.0f);      // quant.py:21-22
#pragma unroll
        for (int k = 0; k < NB; ++k) {
            const uint32_t i = i0 + k * stride;
            if (i < nblocks) scales[i] = (uint8_t)e4m3_byte(rd<MODE>(block_scalar<MODE>(am[k]) / unit));   // quant.py:23
        }
        return unit;
    };
    __syncthreads();                                               // thread 0 is through the tree: sh.last, sh.result
    const uint32_t j = blockIdx.x % kGroups;
    if (!sh.last) {
        // ---- wait for the last workgroup's word, a bounded number of polls
        if (threadIdx.x < 64) {
            uint64_t w = 0;
            uint32_t polls = 0;
            bool have = false;
            for (;;) {
                w = METIS_AT_LOAD(sync_result(sync, j));
                have = is_result(w, tag);
                if (have || ++polls > spin_limit) break;
                __builtin_amdgcn_s_sleep(2);
            }
            if (threadIdx.x == 0) {
                sh.known = have ? 1u : 0u;
                sh.result = __uint_as_float(((uint32_t)w & 0xffffu) << 16);
            }
        }
        __syncthreads();
        if (!sh.known) {
            // ---- leave: park the block maxima, raise the flag, tell the group's word -- unless the result is there by now
#pragma unroll
            for (int k = 0; k < NB; ++k) {
                const uint32_t i = i0 + k * stride;
                if (i < nblocks) parked[i] = (uint16_t)(__float_as_uint(am[k]) >> 16);
            }
            __threadfence();
            __syncthreads();
            if (threadIdx.x == 0) {
                METIS_AT_STORE(sync_left_flag(sync, blockIdx.x), (uint32_t)tag);
                __threadfence();                                   // maxima and flag are out before the marker can be seen
                uint64_t w = METIS_AT_LOAD(sync_result(sync, j));
                for (;;) {
                    if (is_result(w, tag)) {
                        sh.known = 1u;
                        sh.result = __uint_as_float(((uint32_t)w & 0xffffu) << 16);
                        break;
                    }
                    if (is_left_marker(w, tag) || METIS_AT_CAS(sync_result(sync, j), &w, result_word(tag, 1u, 0u))) break;
                }
            }
            __syncthreads();
            if (!sh.known) return;                                 // the last workgroup writes this workgroup's scale bytes
        }
        scale_bytes(sh.result);
        return;
    }
    // ---- the last workgroup to arrive: publish, then look after workgroups that have left
    const float amax = sh.result;
    const uint32_t ngroups = gridDim.x < kGroups ? gridDim.x : kGroups;
    bool somebody_left = false;
    if (threadIdx.x < ngroups)
        somebody_left = is_left_marker(METIS_AT_XCHG(sync_result(sync, threadIdx.x), result_word(tag, 0u, __float_as_uint(amax) >> 16)), tag);
    if (threadIdx.x == 0) sh.nleft = 0u;
    const float unit = scale_bytes(amax);
    if (threadIdx.x == 0) *unit_out = unit;
    if (__syncthreads_or(somebody_left)) {
        __threadfence();                                           // their parked maxima and flags were out before their markers
        for (uint32_t slab = 0; slab < gridDim.x; slab += 256u) {
            const uint32_t b = slab + threadIdx.x;
            if (b < gridDim.x && METIS_AT_LOAD(sync_left_flag(sync, b)) == (uint32_t)tag) sh.left[atomicAdd(&sh.nleft, 1u)] = b;
            __syncthreads();
            const uint32_t nd = sh.nleft;
            for (uint32_t d = 0; d < nd; ++d) {
                const uint32_t base = sh.left[d] * 256u + threadIdx.x;
#pragma unroll
                for (int k = 0; k < NB; ++k) {
                    const uint32_t i = base + k * stride;
                    if (i < nblocks) {
                        const float a = __uint_as_float((uint32_t)parked[i] << 16);
                        scales[i] = (uint8_t)e4m3_byte(rd<MODE>(block_scalar<MODE>(a) / unit));
                    }
                }
            }
            __syncthreads();
            if (threadIdx.x == 0) sh.nleft = 0u;
            __syncthreads();
        }
    }
    if (threadIdx.x == 0) METIS_AT_STORE(sync_generation(sync), tag);
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
// Phase 2 with the dequantized tensor (the round trip of quant.py:6-36: codes, scale bytes AND the dequantized values
// from one call): tensor unit, E4M3 bytes and out = ((v * sign) / 2) * (e4m3 * unit) in one pass over the codes and the
// parked maxima.  A lane owns half a block (one word of codes, 16 bytes of output), so every load and store instruction
// of a wave covers consecutive bytes; the hardware converter turns two codes into their binary32 values (E2M1 = v / 2
// with its sign).  The scale bytes of a wave's 32 blocks leave as eight dwords.
// ---------------------------------------------------------------------------------------------
typedef float metis_f32x2_t __attribute__((ext_vector_type(2)));
template <int MODE>
__global__ __launch_bounds__(256) void quant_scales_dequant_kernel(const uint32_t* __restrict__ codes, const uint16_t* __restrict__ ws_amax,
                                                                   const uint32_t* __restrict__ ws_gmax, uint32_t ngroups,
                                                                   uint8_t* __restrict__ scales, float* __restrict__ unit_out,
                                                                   metis_u32x4_t* __restrict__ out, uint32_t nhalves)
{
    __shared__ float smax[4];
    const uint32_t step = gridDim.x * 256u;
    uint32_t i = blockIdx.x * 256u + threadIdx.x;               // half-block index
    uint32_t cw = 0u, aw = 0u;
    if (i < nhalves) { cw = codes[i]; aw = ws_amax[i >> 1]; }
    float m = 0.0f;
    for (uint32_t g = threadIdx.x; g < ngroups; g += 256u) m = fmaxf(m, __uint_as_float(ws_gmax[g]));
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) smax[threadIdx.x >> 6] = m;
    __syncthreads();
    const float unit = tensor_unit_of<MODE>(fmaxf(fmaxf(smax[0], smax[1]), fmaxf(smax[2], smax[3])));
    if (blockIdx.x == 0 && threadIdx.x == 0) *unit_out = unit;
    const uint32_t lane = threadIdx.x & 63u;
    while (i < nhalves) {
        const uint32_t nxt = i + step;
        uint32_t ncw = 0u, naw = 0u;
        if (nxt < nhalves) { ncw = codes[nxt]; naw = ws_amax[nxt >> 1]; }
        const uint32_t byte = scale_byte_of<MODE>(aw, unit);
        const float dq = rd<MODE>(e4m3_value(byte) * unit);
        uint32_t w[4];
#define METIS_DQ_PAIR(J)                                                                                  \
        {                                                                                                 \
            const metis_f32x2_t v = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(cw, 1.0f, J);                \
            w[J] = rb_pair(rd<MODE>(v.x * dq), rd<MODE>(v.y * dq));                                       \
        }
        METIS_DQ_PAIR(0) METIS_DQ_PAIR(1) METIS_DQ_PAIR(2) METIS_DQ_PAIR(3)
#undef METIS_DQ_PAIR
        __builtin_nontemporal_store((metis_u32x4_t){w[0], w[1], w[2], w[3]}, out + i);
        // scale bytes: the wave's 32 blocks; lane 8 j + {0, 2, 4, 6} hold the bytes of dword j
        const uint32_t b1 = __shfl(byte, (lane & ~7u) + 2u, 64), b2 = __shfl(byte, (lane & ~7u) + 4u, 64), b3 = __shfl(byte, (lane & ~7u) + 6u, 64);
        if ((lane & 7u) == 0u) {
            const uint32_t blk = i >> 1;                          // first of four consecutive blocks
            if (2u * (blk + 3u) < nhalves) *reinterpret_cast<uint32_t*>(scales + blk) = byte | (b1 << 8) | (b2 << 16) | (b3 << 24);
            else {
                const uint32_t bs[4] = {byte, b1, b2, b3};
                for (uint32_t j = 0; j < 4u && 2u * (blk + j) < nhalves; ++j) scales[blk + j] = (uint8_t)bs[j];
            }
        }
        cw = ncw; aw = naw; i = nxt;
    }
}

// ---------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------
static int grid_for(uint32_t work_items, int per_cu = 8)           // 8 workgroups of 256 per CU are resident
{
    int64_t g = ((int64_t)work_items + 255) / 256;
    const int64_t cap = (int64_t)device_cus() * per_cu;
    if (g > cap) g = cap;
    if (g > kMaxGroups) g = kMaxGroups;
    return g < 1 ? 1 : (int)g;
}

int launch_scales_decode(int mode, const Workspace& ws, uint32_t ngroups, const void* codes, void* scales, float* unit, int64_t rows,
                         int64_t cols, void* decode, hipStream_t st)
{
    if (rows <= 0 || rows >= 256 || cols <= 0 || cols % 256 || (mode != METIS_MODE_P32 && mode != METIS_MODE_PB16)) return METIS_E_ARG;
    if (!decode || ((uintptr_t)decode % 16) || ((uintptr_t)scales % 8) || ((uintptr_t)codes % 16)) return METIS_E_ARG;
    const int blocks = (int)(((rows + 31) / 32) * (cols / 256));
    const int cap = device_cus() * 8;
    const dim3 grid((unsigned)(blocks < cap ? blocks : cap));
    if (mode == 0)
        hipLaunchKernelGGL((quant_scales_decode_kernel<0>), grid, dim3(256), 0, st, ws.amax, ws.gmax, ngroups, (const uint8_t*)codes,
                           (uint8_t*)scales, unit, (uint8_t*)decode, (int)rows, (int)cols, blocks);
    else
        hipLaunchKernelGGL((quant_scales_decode_kernel<1>), grid, dim3(256), 0, st, ws.amax, ws.gmax, ngroups, (const uint8_t*)codes,
                           (uint8_t*)scales, unit, (uint8_t*)decode, (int)rows, (int)cols, blocks);
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

int launch_scales(int mode, const Workspace& ws, uint32_t ngroups, void* scales, float* unit, uint32_t nblocks,
                  hipStream_t st, const void* amax2, void* scales2, float* unit2)
{
    const int g2 = grid_for((nblocks + 7) / 8);
    const dim3 grid((unsigned)g2, amax2 ? 2u : 1u);            // a second packing of the same tensor rides in grid row 1
    if (mode == METIS_MODE_P32_F32)
        hipLaunchKernelGGL(quant_scales_f32_kernel, grid, dim3(256), 0, st, (const float*)ws.amax, ws.gmax, ngroups,
                           (uint8_t*)scales, unit, nblocks, (const float*)amax2, (uint8_t*)scales2, unit2);
    else if (mode == 0)
        hipLaunchKernelGGL((quant_scales_kernel<0>), grid, dim3(256), 0, st, ws.amax, ws.gmax, ngroups,
                           (uint8_t*)scales, unit, nblocks, (const uint16_t*)amax2, (uint8_t*)scales2, unit2);
    else
        hipLaunchKernelGGL((quant_scales_kernel<1>), grid, dim3(256), 0, st, ws.amax, ws.gmax, ngroups,
                           (uint8_t*)scales, unit, nblocks, (const uint16_t*)amax2, (uint8_t*)scales2, unit2);
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

// Workgroups per compute unit of the contiguous row quantizer: four waves per SIMD hide the memory latency as well as eight
// do, the last round of blocks (encoded with nothing left to overlap) is half as long, and half as many partial maxima
// are folded later.
constexpr int kContigPerCu = 4;

// Co-resident workgroups of the single-launch kernel on the current device (0 = unknown).
template <int MODE, int NB>
static int fused_capacity()
{
    static int cached[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    if (cached[dev] == 0) {
        int per_cu = 0;
        const hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, quant_fused_kernel<MODE, NB>, 256, 0);
        cached[dev] = (e != hipSuccess || per_cu <= 0) ? -1 : per_cu * device_cus();
    }
    return cached[dev] < 0 ? 0 : cached[dev];
}

template <int MODE, int NB>
static int try_fused(const void* x, void* codes, void* scales, float* unit, const Workspace& ws, uint32_t nblocks,
                     hipStream_t st, uint32_t spin_limit)
{
    int cap = fused_capacity<MODE, NB>();
    if (cap > kFusedMaxGrid) cap = kFusedMaxGrid;
    const int64_t need = ((int64_t)nblocks + 256 * NB - 1) / (256 * NB);
    if (cap <= 0 || need > cap) return 1;                      // does not fit: caller picks another path
    hipLaunchKernelGGL((quant_fused_kernel<MODE, NB>), dim3((unsigned)need), dim3(256), 0, st, (const uint16_t*)x,
                       (uint2*)codes, (uint8_t*)scales, unit, ws.sync, ws.amax, nblocks, spin_limit);
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

template <int MODE>
static int launch_fused(const void* x, void* codes, void* scales, float* unit, const Workspace& ws, uint32_t nblocks,
                        hipStream_t st, uint32_t spin_limit)
{
    int rc = try_fused<MODE, 1>(x, codes, scales, unit, ws, nblocks, st, spin_limit);
    if (rc == 1) rc = try_fused<MODE, 2>(x, codes, scales, unit, ws, nblocks, st, spin_limit);
    if (rc == 1) rc = try_fused<MODE, 4>(x, codes, scales, unit, ws, nblocks, st, spin_limit);
    if (rc == 1) rc = try_fused<MODE, 8>(x, codes, scales, unit, ws, nblocks, st, spin_limit);
    return rc;
}

template <int MODE>
static void launch_contig(const void* x, void* codes, const Workspace& ws, uint32_t nblocks, uint32_t fill_to, int grid, hipStream_t st)
{
    if (measure_int("METIS_Q_DEPTH", 1) == 2)
        hipLaunchKernelGGL((quant_codes_contig_kernel<MODE, 2>), dim3(grid), dim3(256), 0, st, (const uint4*)x, (uint2*)codes, ws.amax,
                           ws.gmax, nblocks, fill_to);
    else
        hipLaunchKernelGGL((quant_codes_contig_kernel<MODE, 1>), dim3(grid), dim3(256), 0, st, (const uint4*)x, (uint2*)codes, ws.amax,
                           ws.gmax, nblocks, fill_to);
}

template <int MODE, bool SR, bool COL, bool WIDE = false, bool HAD = false>
static int launch_quant(const void* x, int64_t rows, int64_t cols, int64_t ld, const void* noise, uint64_t seed,
                        uint64_t offset, void* codes, void* scales, float* unit, const Workspace& ws, hipStream_t st,
                        int in_f32 = 0, const void* center = nullptr, uint32_t sign_mask = 0, void* decode = nullptr)
{
    static_assert(!HAD || !COL, "the rotation runs along the last dimension, as the row blocks do");
    const uint32_t nblocks = (uint32_t)(rows * cols / kBlock);
    if constexpr (COL) {
        const uint32_t tiles_r = (uint32_t)((rows / kBlock + kColTileBlocks - 1) / kColTileBlocks);
        const uint32_t tiles_c = (uint32_t)((cols + kColTileCols - 1) / kColTileCols);
        const int64_t tiles = (int64_t)tiles_r * tiles_c;
        int64_t g = tiles;
        const int64_t cap = (int64_t)device_cus() * 8;
        if (g > cap) g = cap;
        if (g > kMaxGroups) g = kMaxGroups;
        if (WIDE && in_f32)
            hipLaunchKernelGGL((quant_codes_col_kernel<MODE, SR, WIDE, WIDE>), dim3((unsigned)g), dim3(256), 0, st, x,
                               (uint32_t)rows, (uint32_t)cols, ld, noise, seed, offset, (uint2*)codes, (void*)ws.amax, ws.gmax, tiles_c,
                               (uint32_t)tiles, center);
        else
            hipLaunchKernelGGL((quant_codes_col_kernel<MODE, SR, WIDE, false>), dim3((unsigned)g), dim3(256), 0, st, x,
                               (uint32_t)rows, (uint32_t)cols, ld, noise, seed, offset, (uint2*)codes, (void*)ws.amax, ws.gmax, tiles_c,
                               (uint32_t)tiles, center);
        return launch_scales(WIDE ? METIS_MODE_P32_F32 : MODE, ws, (uint32_t)g, scales, unit, nblocks, st);
    } else {
        if constexpr (!SR && !HAD && (WIDE ? MODE == 0 : MODE == 1)) {
            if (center && !in_f32 && ld == cols && cols <= kCentreMaxCols) {   // mean mode on contiguous bf16 rows
                if (decode) return METIS_E_ARG;
                const int gc = grid_for(nblocks, kContigPerCu);
                hipLaunchKernelGGL((quant_codes_contig_centered_kernel<MODE>), dim3(gc), dim3(256), 0, st, (const uint4*)x, center,
                                   (uint2*)codes, (void*)ws.amax, ws.gmax, nblocks, (uint32_t)(cols / kBlock), 0u);
                return launch_scales(WIDE ? METIS_MODE_P32_F32 : MODE, ws, (uint32_t)gc, scales, unit, nblocks, st);
            }
        }
        if constexpr (!SR && !WIDE && !HAD) {
            if (!center && ld == cols) {
                const int gc = grid_for(nblocks, measure_int("METIS_Q_WGPC", kContigPerCu));
                launch_contig<MODE>(x, codes, ws, nblocks, 0u, gc, st);
                if (decode) return launch_scales_decode(MODE, ws, (uint32_t)gc, codes, scales, unit, rows, cols, decode, st);
                return launch_scales(MODE, ws, (uint32_t)gc, scales, unit, nblocks, st);
            }
        }
        if (decode) return METIS_E_ARG;                         // only contiguous bf16 rows, round to nearest, come with the decode layout
        const int g1 = grid_for(nblocks);
        hipLaunchKernelGGL((quant_codes_kernel<MODE, SR, WIDE, HAD>), dim3(g1), dim3(256), 0, st, x, (uint32_t)rows,
                           (uint32_t)cols, ld, noise, seed, offset, (uint2*)codes, (void*)ws.amax, ws.gmax, nblocks, in_f32, center,
                           sign_mask, 0u);
        return launch_scales(WIDE ? METIS_MODE_P32_F32 : MODE, ws, (uint32_t)g1, scales, unit, nblocks, st);
    }
}

int quantize(const void* x, int64_t rows, int64_t cols, int64_t ld, int mode, bool sr, bool col, const void* noise,
             uint64_t seed, uint64_t offset, void* codes, void* scales, float* unit, void* workspace,
             size_t workspace_bytes, hipStream_t st, const void* center, bool resident, uint32_t spin_limit, void* decode)
{
    if (rows < 0 || cols < 0 || ld < cols) return METIS_E_ARG;
    if (mode != METIS_MODE_P32 && mode != METIS_MODE_PB16 && mode != METIS_MODE_P32_F32) return METIS_E_ARG;
    const bool f32in = mode == METIS_MODE_P32_F32;
    if ((col ? rows : cols) % kBlock) return METIS_E_SHAPE;
    if (rows == 0 || cols == 0) return METIS_OK;              // nothing to read or write, unit untouched
    if (!x || !codes || !scales || !unit) return METIS_E_ARG;
    if (rows * cols / kBlock >= (int64_t)1 << 31) return METIS_E_ARG;
    if (!col && ((ld % (f32in ? 4 : 8)) || ((uintptr_t)x % 16))) return METIS_E_ARG;     // 16-byte vector loads
    if (col && f32in && ((uintptr_t)x % 4)) return METIS_E_ARG;
    if (center && ((uintptr_t)center % 16)) return METIS_E_ARG;
    const bool wide = f32in || (center && mode == METIS_MODE_P32);   // a binary32 centre leaves binary32 residuals
    if (((uintptr_t)codes % 8) || ((uintptr_t)scales % 8)) return METIS_E_ARG;
    Workspace ws;
    int rc = carve_workspace(workspace, workspace_bytes, rows, cols, &ws);
    if (rc != METIS_OK) return rc;
    if (decode && (sr || col || wide || center || ld != cols || rows >= 256 || cols % 256)) return METIS_E_ARG;
    if (resident && !decode && !sr && !col && !wide && !center && ld == cols) {   // opt-in single-launch path; falls through when it does not fit
        const uint32_t nblocks = (uint32_t)(rows * cols / kBlock);
        if (spin_limit == 0) spin_limit = kSpinLimit;
        rc = mode == 0 ? launch_fused<0>(x, codes, scales, unit, ws, nblocks, st, spin_limit)
                       : launch_fused<1>(x, codes, scales, unit, ws, nblocks, st, spin_limit);
        if (rc != 1) return rc;
    }
#define METIS_Q(M, S, C) return launch_quant<M, S, C>(x, rows, cols, ld, noise, seed, offset, codes, scales, unit, ws, st, 0, center, 0u, decode)
#define METIS_QF(S, C) return launch_quant<0, S, C, true>(x, rows, cols, ld, noise, seed, offset, codes, scales, unit, ws, st, f32in, center)
    if (wide) {
        if (!sr) { if (!col) METIS_QF(false, false); else METIS_QF(false, true); }
        else { if (!col) METIS_QF(true, false); else METIS_QF(true, true); }
    }
#undef METIS_QF
    if (mode == 0) {
        if (!sr) { if (!col) METIS_Q(0, false, false); else METIS_Q(0, false, true); }
        else { if (!col) METIS_Q(0, true, false); else METIS_Q(0, true, true); }
    } else {
        if (!sr) { if (!col) METIS_Q(1, false, false); else METIS_Q(1, false, true); }
        else { if (!col) METIS_Q(1, true, false); else METIS_Q(1, true, true); }
    }
#undef METIS_Q
}

// The round trip of quant.py:6-36 from one call: codes, scale bytes, unit and the dequantized bf16 tensor, two launches
// (phase 1 as in quantize(); phase 2 forms bytes and dequantized values together).  Contiguous bf16 rows, round to nearest.
int quantize_dequantize_row(const void* x, int64_t rows, int64_t cols, int mode, void* codes, void* scales, float* unit, void* out,
                            void* workspace, size_t workspace_bytes, hipStream_t st)
{
    if (rows < 0 || cols < 0) return METIS_E_ARG;
    if (mode != METIS_MODE_P32 && mode != METIS_MODE_PB16) return METIS_E_ARG;
    if (cols % kBlock) return METIS_E_SHAPE;
    if (rows == 0 || cols == 0) return METIS_OK;
    if (!x || !codes || !scales || !unit || !out) return METIS_E_ARG;
    if (rows * cols / kBlock >= (int64_t)1 << 30) return METIS_E_ARG;
    if (((uintptr_t)x % 16) || ((uintptr_t)out % 16) || ((uintptr_t)codes % 8) || ((uintptr_t)scales % 8)) return METIS_E_ARG;
    Workspace ws;
    if (const int rc = carve_workspace(workspace, workspace_bytes, rows, cols, &ws)) return rc;
    const uint32_t nblocks = (uint32_t)(rows * cols / kBlock);
    const int g1 = grid_for(nblocks, kContigPerCu);
    if (mode == 0) launch_contig<0>(x, codes, ws, nblocks, 0u, g1, st);
    else launch_contig<1>(x, codes, ws, nblocks, 0u, g1, st);
    if (hipGetLastError() != hipSuccess) return METIS_E_LAUNCH;
    const uint32_t nhalves = nblocks * 2u;
    // whole waves of 32 blocks per iteration: the stride is a multiple of 64 halves by construction (256 threads)
    const int g2 = grid_for((nhalves + 3) / 4);                 // four halves per thread
    if (mode == 0)
        hipLaunchKernelGGL((quant_scales_dequant_kernel<0>), dim3(g2), dim3(256), 0, st, (const uint32_t*)codes, ws.amax, ws.gmax, (uint32_t)g1,
                           (uint8_t*)scales, unit, (metis_u32x4_t*)out, nhalves);
    else
        hipLaunchKernelGGL((quant_scales_dequant_kernel<1>), dim3(g2), dim3(256), 0, st, (const uint32_t*)codes, ws.amax, ws.gmax, (uint32_t)g1,
                           (uint8_t*)scales, unit, (metis_u32x4_t*)out, nhalves);
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

// Workgroups of quant_codes_both_kernel that the current device holds at once (its LDS slabs bound them): the grid is
// no larger, so that every workgroup starts at once and walks the same number of tiles, give or take one.
template <int MODE, bool WIDE>
static int both_capacity()
{
    static int cached[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    if (cached[dev] == 0) {
        int per_cu = 0;
        const hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, quant_codes_both_kernel<MODE, WIDE>, 256, 0);
        cached[dev] = (e != hipSuccess || per_cu <= 0) ? -1 : per_cu * device_cus();
    }
    return cached[dev] < 0 ? device_cus() * 4 : cached[dev];
}

// ---------------------------------------------------------------------------------------------
// Both packings of one tensor (rows and columns) with stochastic rounding, one pass over x; then phase 2 for each.
// The workspace holds two areas of parked maxima: 2 x workspace_bytes(rows, cols).
// ---------------------------------------------------------------------------------------------
int quantize_both_sr(const void* x, int64_t rows, int64_t cols, int64_t ld, int mode, uint64_t seed, uint64_t offset_row,
                     uint64_t offset_col, void* codes_row, void* scales_row, float* unit_row, void* codes_col, void* scales_col,
                     float* unit_col, void* workspace, size_t bytes, hipStream_t st)
{
    if (rows < 0 || cols < 0 || ld < cols) return METIS_E_ARG;
    if (mode != METIS_MODE_P32 && mode != METIS_MODE_PB16 && mode != METIS_MODE_P32_F32) return METIS_E_ARG;
    const bool f32in = mode == METIS_MODE_P32_F32;
    if (rows % kBlock || cols % kBlock) return METIS_E_SHAPE;
    if (rows == 0 || cols == 0) return METIS_OK;
    if (!x || !codes_row || !scales_row || !unit_row || !codes_col || !scales_col || !unit_col) return METIS_E_ARG;
    if (rows * cols / kBlock >= (int64_t)1 << 31) return METIS_E_ARG;
    if ((ld % (f32in ? 4 : 8)) || ((uintptr_t)x % 16)) return METIS_E_ARG;                 // 16-byte vector loads
    if (((uintptr_t)codes_row % 8) || ((uintptr_t)scales_row % 8) || ((uintptr_t)codes_col % 8) || ((uintptr_t)scales_col % 8)) return METIS_E_ARG;
    const size_t one = workspace_bytes(rows, cols);
    if (!workspace || ((uintptr_t)workspace % 256) || bytes < 2 * one) return METIS_E_WORKSPACE;
    Workspace wr, wc;
    if (const int rc = carve_workspace(workspace, one, rows, cols, &wr)) return rc;
    if (const int rc = carve_workspace(static_cast<char*>(workspace) + one, one, rows, cols, &wc)) return rc;
    wc.gmax = wr.gmax;                                         // one tensor, one maximum: both packings fold the same partials
    const uint32_t nblocks = (uint32_t)(rows * cols / kBlock);
    const uint32_t tiles_r = (uint32_t)((rows / kBlock + kColTileBlocks - 1) / kColTileBlocks);
    const uint32_t tiles_c = (uint32_t)((cols + kColTileCols - 1) / kColTileCols);
    const int64_t tiles = (int64_t)tiles_r * tiles_c;
    int64_t g = tiles;
    const int64_t cap = f32in ? both_capacity<0, true>() : mode == 0 ? both_capacity<0, false>() : both_capacity<1, false>();
    if (g > cap) g = cap;
    if (g > kMaxGroups) g = kMaxGroups;
#define METIS_QB(M, W) hipLaunchKernelGGL((quant_codes_both_kernel<M, W>), dim3((unsigned)g), dim3(256), 0, st, x, (uint32_t)rows, \
                                          (uint32_t)cols, ld, seed, offset_row, offset_col, (uint2*)codes_row, (void*)wr.amax, (uint2*)codes_col, \
                                          (void*)wc.amax, wr.gmax, tiles_c, (uint32_t)tiles)
    if (f32in) METIS_QB(0, true);
    else if (mode == 0) METIS_QB(0, false);
    else METIS_QB(1, false);
#undef METIS_QB
    if (hipGetLastError() != hipSuccess) return METIS_E_LAUNCH;
    const int pm = f32in ? METIS_MODE_P32_F32 : mode;
    return launch_scales(pm, wr, (uint32_t)g, scales_row, unit_row, nblocks, st, wc.amax, scales_col, unit_col);   // one launch for both
}

// ---------------------------------------------------------------------------------------------
// Deferred scale bytes.  The codes of a block depend on the block alone, the scale bytes on the tensor maximum: a
// consumer that runs after the quantizer anyway (the tiled expansion ahead of a GEMM) can form them from the parked
// block maxima, and the quantizer is then ONE launch.  The caller owns the parked data: [0, 8 KiB) the partial maxima
// (kDeferredPartials entries), then one bf16 maximum per block.  Round-to-nearest rows of a contiguous bf16 tensor.
// ---------------------------------------------------------------------------------------------
size_t deferred_bytes(int64_t rows, int64_t cols)
{
    if (rows <= 0 || cols <= 0) return 0;
    const size_t nblocks = (size_t)((rows * cols + 15) / 16);
    return kDeferredPartials * 4 + ((nblocks * 2 + 255) / 256) * 256;
}

int carve_deferred(void* p, size_t bytes, int64_t rows, int64_t cols, Workspace* ws)
{
    if (!p || ((uintptr_t)p % 256) || bytes < deferred_bytes(rows, cols)) return METIS_E_WORKSPACE;
    ws->gmax = static_cast<uint32_t*>(p);
    ws->sync = nullptr;
    ws->amax = reinterpret_cast<uint16_t*>(static_cast<char*>(p) + kDeferredPartials * 4);
    return METIS_OK;
}

int deferred_grid(uint32_t work_items, int per_cu)
{
    const int g = grid_for(work_items, per_cu);
    return g > (int)kDeferredPartials ? (int)kDeferredPartials : g;
}

// center (bf16 arithmetic only: a binary32 centre leaves residuals whose maxima are not bf16 values): one bf16 value per
// column subtracted first, as quantize() does for the mean mode.
int quantize_row_deferred(const void* x, int64_t rows, int64_t cols, int mode, const void* center, void* codes, void* deferred,
                          size_t bytes, hipStream_t st)
{
    if (rows < 0 || cols < 0) return METIS_E_ARG;
    if (mode != METIS_MODE_P32 && mode != METIS_MODE_PB16) return METIS_E_ARG;
    if (center && (mode != METIS_MODE_PB16 || ((uintptr_t)center % 16))) return METIS_E_ARG;
    if (cols % kBlock) return METIS_E_SHAPE;
    if (rows == 0 || cols == 0) return METIS_OK;
    if (!x || !codes || ((uintptr_t)x % 16) || ((uintptr_t)codes % 8)) return METIS_E_ARG;
    if (rows * cols / kBlock >= (int64_t)1 << 31) return METIS_E_ARG;
    Workspace ws;
    if (const int rc = carve_deferred(deferred, bytes, rows, cols, &ws)) return rc;
    const uint32_t nblocks = (uint32_t)(rows * cols / kBlock);
    const int g1 = deferred_grid(nblocks, center ? 8 : measure_int("METIS_Q_WGPC", kContigPerCu));
    if (center && cols <= kCentreMaxCols)
        hipLaunchKernelGGL((quant_codes_contig_centered_kernel<1>), dim3(g1), dim3(256), 0, st, (const uint4*)x, center, (uint2*)codes,
                           (void*)ws.amax, ws.gmax, nblocks, (uint32_t)(cols / kBlock), kDeferredPartials);
    else if (center)
        hipLaunchKernelGGL((quant_codes_kernel<1, false, false, false>), dim3(g1), dim3(256), 0, st, x, (uint32_t)rows, (uint32_t)cols,
                           cols, nullptr, (uint64_t)0, (uint64_t)0, (uint2*)codes, (void*)ws.amax, ws.gmax, nblocks, 0, center, 0u,
                           kDeferredPartials);
    else if (mode == 0)
        launch_contig<0>(x, codes, ws, nblocks, kDeferredPartials, g1, st);
    else
        launch_contig<1>(x, codes, ws, nblocks, kDeferredPartials, g1, st);
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

// quantize_row_deferred of a decode-sized contiguous bf16 activation and, in the same launch, the first step of its
// rank-r projection onto v [R, cols]: partial sums per K chunk into lr_workspace (lowrank_small's workspace), for a
// finishing step that runs later (decode_prepare_deferred with x = nullptr).
int quantize_row_deferred_partial(const void* x, int64_t rows, int64_t cols, int mode, void* codes, void* deferred, size_t bytes,
                                  const void* v, int64_t R, void* lr_workspace, size_t lr_workspace_bytes, hipStream_t st)
{
    if (rows < 0 || cols < 0 || R <= 0) return METIS_E_ARG;
    if (mode != METIS_MODE_P32 && mode != METIS_MODE_PB16) return METIS_E_ARG;
    if (rows == 0 || rows >= 256 || cols == 0 || cols % 64 || R % 32 || R > 128) return METIS_E_SHAPE;
    if (!x || !codes || !v || ((uintptr_t)x % 16) || ((uintptr_t)codes % 8) || ((uintptr_t)v % 16)) return METIS_E_ARG;
    if (!lr_workspace || ((uintptr_t)lr_workspace % 16) || lr_workspace_bytes < lowrank_small_workspace_bytes(rows, R, cols))
        return METIS_E_WORKSPACE;
    Workspace ws;
    if (const int rc = carve_deferred(deferred, bytes, rows, cols, &ws)) return rc;
    const uint32_t nblocks = (uint32_t)(rows * cols / kBlock);
    const int g1 = deferred_grid(nblocks, kContigPerCu);
    int kc;
    const int chunks = lowrank_small_chunks(cols, &kc);
    const int g = g1 + chunks * (int)((rows + 63) / 64);
#define METIS_QP(MODE) hipLaunchKernelGGL((decode_quant_partial_kernel<MODE>), dim3(g), dim3(256), 0, st, (uint32_t)g1, (const uint4*)x, \
                                          (uint2*)codes, ws.amax, ws.gmax, nblocks, kDeferredPartials, cols, (const uint16_t*)v, \
                                          (int)rows, (int)R, (int)cols, kc, chunks, (float*)lr_workspace)
    if (mode == 0) METIS_QP(0); else METIS_QP(1);
#undef METIS_QP
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

// phase 2 on parked data, whenever somebody wants the bytes after all
int deferred_scales(const void* deferred, int64_t rows, int64_t cols, int mode, void* scales, float* unit, hipStream_t st)
{
    if (rows < 0 || cols < 0 || (mode != METIS_MODE_P32 && mode != METIS_MODE_PB16)) return METIS_E_ARG;
    if (cols % kBlock) return METIS_E_SHAPE;
    if (rows == 0 || cols == 0) return METIS_OK;
    if (!scales || !unit || ((uintptr_t)scales % 8)) return METIS_E_ARG;
    Workspace ws;
    if (const int rc = carve_deferred(const_cast<void*>(deferred), deferred_bytes(rows, cols), rows, cols, &ws)) return rc;
    return launch_scales(mode, ws, kDeferredPartials, scales, unit, (uint32_t)(rows * cols / kBlock), st);
}

// ---------------------------------------------------------------------------------------------
// "svd" mode of the activation / output-gradient decomposition (src/Metis/Metis/bitlinear.py:283-303): the tensor that is
// quantized is x - ker with ker = (U diag(s)) V of rank r, and the caller goes on with ker + QDQ(x - ker).  ker is formed
// in registers: a workgroup owns tiles of 64 rows x 256 columns, a thread one block of 16 columns in four rows, and the
// factors pass through LDS sixteen ranks at a time.  Every element of ker is the chain
//     acc = 0;  acc = fma(us[i][k], v[k][j], acc)  for k = 0 .. r-1 in that order, in binary32
// (bf16 arithmetic: exact products of bf16 factors, the sum rounded to bf16 once, as a bf16 matrix product with
// binary32 accumulation does) -- a fixed order, so that a CPU restatement reproduces the bits.  Then the residual
// x - ker (rounded to the arithmetic's type) is encoded like any other block; the codes and the parked block maxima go
// where the row quantizer puts them, and ker is written out only when the caller wants the dense result.
// ---------------------------------------------------------------------------------------------
constexpr int kLrRows = 64, kLrCols = 256, kLrRanks = 16;

template <int MODE, bool F32IN>
__global__ __launch_bounds__(256) void quant_lowrank_residual_kernel(
    const void* __restrict__ xv, const void* __restrict__ usv, const void* __restrict__ vtv, uint32_t rows, uint32_t cols,
    uint32_t rank, uint2* __restrict__ codes, void* __restrict__ ws_amax_v, uint32_t* __restrict__ ws_gmax,
    void* __restrict__ ker_out, uint32_t tiles_c, uint32_t tiles)
{
    static_assert(MODE == 0 || !F32IN, "bf16 arithmetic reads bf16 tensors");
    // LDS layouts without bank conflicts: of V, quarter q of every thread's block of 16 lies side by side with the same
    // quarter of the fifteen other blocks (a 16-byte read of sixteen lanes covers 256 contiguous bytes); the rows of
    // U diag(s) are 80 bytes apart, so that the four row groups of a wave read from different banks.
    __shared__ float4 s_v[kLrRanks][4][kLrCols / kBlock];
    __shared__ __align__(16) float s_u[kLrRows][kLrRanks + 4];
    const uint32_t t = threadIdx.x, cb = t & 15u, rg = t >> 4;
    const uint32_t nbpr = cols / kBlock;
    float gmax = 0.0f;
    for (uint32_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
        const uint32_t tr = tile / tiles_c, tc = tile - tr * tiles_c;
        const uint32_t row0 = tr * kLrRows, col0 = tc * kLrCols;
        float acc[4][kBlock];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < kBlock; ++j) acc[i][j] = 0.0f;
        // The factors of the next sixteen ranks are fetched into registers while the current ones are multiplied, and go to
        // LDS between two barriers afterwards: their memory latency is off the critical path.
        float pv[kBlock];
        float4 pu;
        auto fetch_chunk = [&](uint32_t k0) {
            {   // V: rank k0 + t / 16, columns col0 + 16 (t % 16) ..; zeros beyond the tensor
                const uint32_t k = k0 + rg, c = col0 + cb * kBlock;
#pragma unroll
                for (int j = 0; j < kBlock; ++j) pv[j] = 0.0f;
                if (c < cols) {
                    if constexpr (MODE == 0) {
                        const float4* p = reinterpret_cast<const float4*>(static_cast<const float*>(vtv) + (size_t)k * cols + c);
#pragma unroll
                        for (int q = 0; q < 4; ++q) { const float4 f = p[q]; pv[4 * q] = f.x; pv[4 * q + 1] = f.y; pv[4 * q + 2] = f.z; pv[4 * q + 3] = f.w; }
                    } else {
                        const uint4* p = reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(vtv) + (size_t)k * cols + c);
                        unpack16(p[0], p[1], pv);
                    }
                }
            }
            {   // U diag(s): row row0 + t / 4, ranks k0 + 4 (t % 4) ..
                const uint32_t r = row0 + (t >> 2), k = k0 + (t & 3u) * 4u;
                pu = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                if (r < rows) {
                    if constexpr (MODE == 0) pu = *reinterpret_cast<const float4*>(static_cast<const float*>(usv) + (size_t)r * rank + k);
                    else {
                        const uint2 w = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(usv) + (size_t)r * rank + k);
                        pu = make_float4(bf16_lo(w.x), bf16_hi(w.x), bf16_lo(w.y), bf16_hi(w.y));
                    }
                }
            }
        };
        fetch_chunk(0);
        for (uint32_t k0 = 0; k0 < rank; k0 += kLrRanks) {
            __syncthreads();                                   // the previous chunk (or tile) has been read
            {
#pragma unroll
                for (int q = 0; q < 4; ++q) s_v[rg][q][cb] = make_float4(pv[4 * q], pv[4 * q + 1], pv[4 * q + 2], pv[4 * q + 3]);
                *reinterpret_cast<float4*>(&s_u[t >> 2][(t & 3u) * 4u]) = pu;
            }
            __syncthreads();
            if (k0 + kLrRanks < rank) fetch_chunk(k0 + kLrRanks);
#pragma unroll
            for (int kq = 0; kq < kLrRanks / 4; ++kq) {
                float4 u4[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) u4[i] = *reinterpret_cast<const float4*>(&s_u[rg * 4 + i][kq * 4]);
#pragma unroll
                for (int kk = 0; kk < 4; ++kk) {
                    float vv[kBlock];
#pragma unroll
                    for (int q = 0; q < 4; ++q) { const float4 f = s_v[kq * 4 + kk][q][cb]; vv[4 * q] = f.x; vv[4 * q + 1] = f.y; vv[4 * q + 2] = f.z; vv[4 * q + 3] = f.w; }
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float uu = kk == 0 ? u4[i].x : kk == 1 ? u4[i].y : kk == 2 ? u4[i].z : u4[i].w;
#pragma unroll
                        for (int j = 0; j < kBlock; ++j) acc[i][j] = fmaf(uu, vv[j], acc[i][j]);
                    }
                }
            }
        }
        const uint32_t cbg = tc * (kLrCols / kBlock) + cb;      // block column in the tensor
        if (cbg < nbpr) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t row = row0 + rg * 4u + (uint32_t)i;
                if (row >= rows) break;
                const size_t e0 = (size_t)row * cols + (size_t)cbg * kBlock;
                float v[kBlock];
                if constexpr (F32IN) {
                    const float4* p = reinterpret_cast<const float4*>(static_cast<const float*>(xv) + e0);
#pragma unroll
                    for (int q = 0; q < 4; ++q) { const float4 f = p[q]; v[4 * q] = f.x; v[4 * q + 1] = f.y; v[4 * q + 2] = f.z; v[4 * q + 3] = f.w; }
                } else {
                    const uint4* p = reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(xv) + e0);
                    unpack16(p[0], p[1], v);
                }
                if constexpr (MODE == 0) {
                    if (ker_out) {
                        float4* o = reinterpret_cast<float4*>(static_cast<float*>(ker_out) + e0);
#pragma unroll
                        for (int q = 0; q < 4; ++q) o[q] = make_float4(acc[i][4 * q], acc[i][4 * q + 1], acc[i][4 * q + 2], acc[i][4 * q + 3]);
                    }
#pragma unroll
                    for (int j = 0; j < kBlock; ++j) v[j] -= acc[i][j];
                } else {
                    uint32_t kw[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) kw[j] = bf16_bits(acc[i][2 * j]) | (bf16_bits(acc[i][2 * j + 1]) << 16);
                    if (ker_out) {
                        uint4* o = reinterpret_cast<uint4*>(static_cast<uint16_t*>(ker_out) + e0);
                        o[0] = make_uint4(kw[0], kw[1], kw[2], kw[3]);
                        o[1] = make_uint4(kw[4], kw[5], kw[6], kw[7]);
                    }
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        v[2 * j] = rb(v[2 * j] - bf16_lo(kw[j]));
                        v[2 * j + 1] = rb(v[2 * j + 1] - bf16_hi(kw[j]));
                    }
                }
                const float am = block_amax(v);
                gmax = fmaxf(gmax, am);
                const uint32_t blk = row * nbpr + cbg;
                if constexpr (MODE == 0) {
                    static_cast<float*>(ws_amax_v)[blk] = am;
                    codes[blk] = encode_rne_wide(v, block_scalar_ieee(am));
                } else {
                    const float none[kBlock] = {};
                    static_cast<uint16_t*>(ws_amax_v)[blk] = (uint16_t)(__float_as_uint(am) >> 16);
                    codes[blk] = encode_block<1, false>(v, block_scalar<1>(am), none);
                }
            }
        }
    }
    publish_group_max(gmax, ws_gmax, 0u);
}

// out = ker + QDQ(x - ker), in place on the buffer that holds ker (bitlinear.py:301-303): eight elements per thread
template <int MODE>
__global__ __launch_bounds__(256) void lowrank_add_dequant_kernel(const uint32_t* __restrict__ codes, const uint8_t* __restrict__ scales,
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
            float v = (float)(r + (r > 4u ? r - 4u : 0u) + (r > 6u ? 2u * (r - 6u) : 0u));
            v = (nib & 8u) ? -v : v;
            o[j] = rd<MODE>((v * 0.5f) * dq);
        }
        if constexpr (MODE == 0) {
            float4* p = reinterpret_cast<float4*>(out) + i * 2;
            const float4 a = p[0], b = p[1];
            p[0] = make_float4(a.x + o[0], a.y + o[1], a.z + o[2], a.w + o[3]);
            p[1] = make_float4(b.x + o[4], b.y + o[5], b.z + o[6], b.w + o[7]);
        } else {
            uint4* p = reinterpret_cast<uint4*>(out) + i;
            const uint4 k = *p;
            uint4 w;
            w.x = rb_pair(bf16_lo(k.x) + o[0], bf16_hi(k.x) + o[1]);
            w.y = rb_pair(bf16_lo(k.y) + o[2], bf16_hi(k.y) + o[3]);
            w.z = rb_pair(bf16_lo(k.z) + o[4], bf16_hi(k.z) + o[5]);
            w.w = rb_pair(bf16_lo(k.w) + o[6], bf16_hi(k.w) + o[7]);
            *p = w;
        }
    }
}

int quantize_lowrank_residual(const void* x, bool x_f32, const void* us, const void* vt, int64_t rows, int64_t cols, int rank, int mode,
                              void* codes, void* scales, float* unit, void* dense, void* workspace, size_t workspace_bytes,
                              hipStream_t st)
{
    if (rows < 0 || cols < 0 || rank <= 0) return METIS_E_ARG;
    if (mode != METIS_MODE_P32 && mode != METIS_MODE_PB16) return METIS_E_ARG;
    if (x_f32 && mode != METIS_MODE_P32) return METIS_E_ARG;
    if (cols % kBlock || rank % kLrRanks) return METIS_E_SHAPE;
    if (rows == 0 || cols == 0) return METIS_OK;
    if (!x || !us || !vt || !codes || !scales || !unit) return METIS_E_ARG;
    if (((uintptr_t)x % 16) || ((uintptr_t)us % 16) || ((uintptr_t)vt % 16) || ((uintptr_t)dense % 16) || ((uintptr_t)codes % 8) ||
        ((uintptr_t)scales % 8))
        return METIS_E_ARG;
    if (rows * cols / kBlock >= (int64_t)1 << 31) return METIS_E_ARG;
    Workspace ws;
    if (const int rc = carve_workspace(workspace, workspace_bytes, rows, cols, &ws)) return rc;
    const uint32_t tiles_c = (uint32_t)((cols + kLrCols - 1) / kLrCols);
    const int64_t tiles = (int64_t)((rows + kLrRows - 1) / kLrRows) * tiles_c;
    int64_t g = tiles;
    if (g > (int64_t)device_cus() * 3) g = (int64_t)device_cus() * 3;          // three workgroups per CU are resident (139 VGPRs)
    if (g > kMaxGroups) g = kMaxGroups;
    const uint32_t nblocks = (uint32_t)(rows * cols / kBlock);
#define METIS_LR(M, F)                                                                                                          \
    hipLaunchKernelGGL((quant_lowrank_residual_kernel<M, F>), dim3((unsigned)g), dim3(256), 0, st, x, us, vt, (uint32_t)rows,      \
                       (uint32_t)cols, (uint32_t)rank, (uint2*)codes, (void*)ws.amax, ws.gmax, dense, tiles_c, (uint32_t)tiles)
    if (mode == METIS_MODE_PB16) METIS_LR(1, false);
    else if (x_f32) METIS_LR(0, true);
    else METIS_LR(0, false);
#undef METIS_LR
    if (hipGetLastError() != hipSuccess) return METIS_E_LAUNCH;
    if (const int rc = launch_scales(mode == METIS_MODE_P32 ? METIS_MODE_P32_F32 : METIS_MODE_PB16, ws, (uint32_t)g, scales, unit, nblocks, st,
                                     nullptr, nullptr, nullptr))
        return rc;
    if (dense) {
        const int64_t noct = rows * cols / 8;
        const int g3 = grid_for((uint32_t)noct);                 // noct < 2^32: nblocks < 2^31
        if (mode == METIS_MODE_P32)
            hipLaunchKernelGGL((lowrank_add_dequant_kernel<0>), dim3(g3), dim3(256), 0, st, (const uint32_t*)codes, (const uint8_t*)scales, unit, dense, noct);
        else
            hipLaunchKernelGGL((lowrank_add_dequant_kernel<1>), dim3(g3), dim3(256), 0, st, (const uint32_t*)codes, (const uint8_t*)scales, unit, dense, noct);
        if (hipGetLastError() != hipSuccess) return METIS_E_LAUNCH;
    }
    return METIS_OK;
}

// ---------------------------------------------------------------------------------------------
// NV recipe: rotate every tile of 16 along the last dimension, then quantize the rotated tensor (row blocks = tiles),
// in one pass over x.  Round to nearest, or stochastic rounding on the library's own stream.
// ---------------------------------------------------------------------------------------------
int quantize_rht(const void* x, int64_t rows, int64_t cols, int64_t ld, int mode, uint32_t sign_mask, bool sr, uint64_t seed,
                 uint64_t offset, void* codes, void* scales, float* unit, void* workspace, size_t workspace_bytes, hipStream_t st)
{
    if (rows < 0 || cols < 0 || ld < cols || sign_mask > 0xffffu) return METIS_E_ARG;
    if (mode != METIS_MODE_P32 && mode != METIS_MODE_PB16 && mode != METIS_MODE_P32_F32) return METIS_E_ARG;
    const bool f32in = mode == METIS_MODE_P32_F32;
    if (cols % kBlock) return METIS_E_SHAPE;
    if (rows == 0 || cols == 0) return METIS_OK;
    if (!x || !codes || !scales || !unit) return METIS_E_ARG;
    if (rows * cols / kBlock >= (int64_t)1 << 31) return METIS_E_ARG;
    if ((ld % (f32in ? 4 : 8)) || ((uintptr_t)x % 16)) return METIS_E_ARG;
    if (((uintptr_t)codes % 8) || ((uintptr_t)scales % 8)) return METIS_E_ARG;
    Workspace ws;
    if (const int rc = carve_workspace(workspace, workspace_bytes, rows, cols, &ws)) return rc;
#define METIS_QH(M, S, W) return launch_quant<M, S, false, W, true>(x, rows, cols, ld, nullptr, seed, offset, codes, scales, unit, ws, st, \
                                                                    f32in, nullptr, sign_mask)
    if (mode == METIS_MODE_PB16) { if (sr) METIS_QH(1, true, false); else METIS_QH(1, false, false); }
    if (sr) METIS_QH(0, true, true); else METIS_QH(0, false, true);
#undef METIS_QH
}

// The rotation alone, bf16 or binary32 in and out (same dtype): out = rotate(x) or its inverse, tile by tile.
template <int F32, int INVERSE>
__global__ __launch_bounds__(256) void hadamard16_kernel(const void* __restrict__ xv, void* __restrict__ outv, int64_t ntiles,
                                                         int64_t tiles_per_row, int64_t ldx, int64_t ldo, uint32_t sign_mask)
{
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < ntiles; i += (int64_t)gridDim.x * 256) {
        const int64_t row = i / tiles_per_row, cb = i - row * tiles_per_row;
        float v[kBlock];
        if (F32) {
            const float4* p = reinterpret_cast<const float4*>(static_cast<const float*>(xv) + row * ldx + cb * kBlock);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const float4 f = p[c];
                v[4 * c] = f.x; v[4 * c + 1] = f.y; v[4 * c + 2] = f.z; v[4 * c + 3] = f.w;
            }
        } else {
            const uint4* p = reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(xv) + row * ldx + cb * kBlock);
            unpack16(p[0], p[1], v);
        }
        if (INVERSE) hadamard16_inverse(v, sign_mask);
        else hadamard16_forward(v, sign_mask);
        if (F32) {
            float4* o = reinterpret_cast<float4*>(static_cast<float*>(outv) + row * ldo + cb * kBlock);
#pragma unroll
            for (int c = 0; c < 4; ++c) o[c] = make_float4(v[4 * c], v[4 * c + 1], v[4 * c + 2], v[4 * c + 3]);
        } else {
            uint32_t w[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) w[j] = bf16_bits(v[2 * j]) | (bf16_bits(v[2 * j + 1]) << 16);
            uint4* o = reinterpret_cast<uint4*>(static_cast<uint16_t*>(outv) + row * ldo + cb * kBlock);
            o[0] = make_uint4(w[0], w[1], w[2], w[3]);
            o[1] = make_uint4(w[4], w[5], w[6], w[7]);
        }
    }
}

int hadamard16(const void* x, int64_t rows, int64_t cols, int64_t ldx, int dtype, int inverse, uint32_t sign_mask, void* out,
               int64_t ldo, hipStream_t st)
{
    if (rows < 0 || cols < 0 || ldx < cols || ldo < cols || sign_mask > 0xffffu) return METIS_E_ARG;
    if (dtype != METIS_DTYPE_BF16 && dtype != METIS_DTYPE_F32) return METIS_E_ARG;
    if (cols % kBlock) return METIS_E_SHAPE;
    if (rows == 0 || cols == 0) return METIS_OK;
    const int al = dtype == METIS_DTYPE_F32 ? 4 : 8;
    if (!x || !out || (ldx % al) || (ldo % al) || ((uintptr_t)x % 16) || ((uintptr_t)out % 16)) return METIS_E_ARG;
    const int64_t tpr = cols / kBlock, ntiles = rows * tpr;
    int64_t g = (ntiles + 255) / 256;
    const int64_t cap = (int64_t)device_cus() * 16;
    if (g > cap) g = cap;
#define METIS_H(F, I) hipLaunchKernelGGL((hadamard16_kernel<F, I>), dim3((unsigned)g), dim3(256), 0, st, x, out, ntiles, tpr, ldx, ldo, sign_mask)
    if (dtype == METIS_DTYPE_F32) { if (inverse) METIS_H(1, 1); else METIS_H(1, 0); }
    else { if (inverse) METIS_H(0, 1); else METIS_H(0, 0); }
#undef METIS_H
    return hipGetLastError() == hipSuccess ? METIS_OK : METIS_E_LAUNCH;
}

// ---------------------------------------------------------------------------------------------
// Allocation-free variant of the row quantizer: the workspace (per-workgroup maxima, reduction words,
// parked block maxima) is a file-scope device array instead of caller memory, for callers that cannot
// allocate (HIP graph capture, serving loops).  Every device the library runs on holds its own copy of
// the array at its own address until the process ends; the address is looked up once per device, with
// that device current, and host code only ever uses that address, never the array's name.
// ---------------------------------------------------------------------------------------------
constexpr int64_t kStaticMaxElements = (int64_t)1 << 26;         // 64 Mi elements, e.g. [16384, 4096]
constexpr size_t kStaticScratchBytes = kWsGmaxBytes + kWsSyncBytes + (size_t)(kStaticMaxElements / kBlock) * 4;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

static int static_scratch(void** out)
{
    static std::atomic<void*> ptrs[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return METIS_E_DEVICE;
    void* p = ptrs[dev].load(std::memory_order_acquire);
    if (!p) {
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) {
            (void)hipGetLastError();
            return METIS_E_DEVICE;
        }
        ptrs[dev].store(p, std::memory_order_release);         // two racing first calls store the same address
    }
    *out = p;
    return METIS_OK;
}

int quantize_row_static(const void* x, int64_t rows, int64_t cols, int64_t ld, int mode, void* codes, void* scales,
                        float* unit, hipStream_t st)
{
    if (rows < 0 || cols < 0) return METIS_E_ARG;
    if (mode != METIS_MODE_P32 && mode != METIS_MODE_PB16 && mode != METIS_MODE_P32_F32) return METIS_E_ARG;
    if (rows > 0 && cols > kStaticMaxElements / rows) return METIS_E_TOO_LARGE;
    static_assert(kStaticScratchBytes >= kWsGmaxBytes + kWsSyncBytes + (size_t)(kStaticMaxElements / kBlock) * 4, "scratch too small");
    void* ws = nullptr;
    if (const int rc = static_scratch(&ws)) return rc;
    // the two-launch path: nothing in the scratch has to start at zero (phase 1 rewrites every word phase 2 reads)
    return quantize(x, rows, cols, ld, mode, false, false, nullptr, 0, 0, codes, scales, unit, ws, kStaticScratchBytes, st);
}

int dequantize(const void* codes, const void* scales, const float* unit, int64_t rows, int64_t cols, int mode, void* out,
               int out_dtype, hipStream_t st)
{
    if (rows < 0 || cols < 0) return METIS_E_ARG;
    if (mode == METIS_MODE_P32_F32) mode = METIS_MODE_P32;     // same arithmetic, the packed format does not know its source
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
