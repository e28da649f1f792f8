// Per-block NVFP4 encoding shared by the quantizer kernels (plain and RMSNorm-fused).
#pragma once
#include "metis_device.h"
#include "quotient_table.h"

namespace metis {

// ---------------------------------------------------------------------------------------------
// E2M1 codes of one block.  v: the 16 elements, s: raw block scalar, u: uniform draws (SR only).
// Packed as two dwords, element 2j in the low nibble of byte j.
// ---------------------------------------------------------------------------------------------
template <int MODE, bool SR>
__device__ __forceinline__ uint2 encode_literal(const float (&v)[kBlock], float s, const float (&u)[kBlock])
{
    const float h = rd<MODE>(s / 2.0f);
    uint32_t w[2] = {0u, 0u};
#pragma unroll
    for (int j = 0; j < kBlock; ++j) {
        float r = code_literal<MODE, SR>(fabsf(v[j]), h, SR ? u[j] : 0.0f);
        uint32_t code = (uint32_t)fminf(fmaxf(r, 0.0f), 7.0f);      // SR may reach 8: clamp to the grid
        code |= (v[j] < 0.0f) ? 8u : 0u;
        w[j >> 3] |= code << (4 * (j & 7));
    }
    return make_uint2(w[0], w[1]);
}

// Round-to-nearest, binary32 arithmetic.  The reference's compress/round/expand sequence equals
// a round-to-nearest-even conversion of q = RN(|x|/h) onto the E2M1 grid for every binary32 q
// except q = 5+1ulp, 7-1ulp and 10+1ulp (exhaustive host check), where its second rounding lands
// on a tie.  The hardware FP4 converter does the RNE conversion two elements at a time on the
// quotient x/s from div3(); a block whose scalar could produce one of the three exceptional
// quotients from a bf16 input, or for which div3() is not provably decisive at a threshold,
// takes the literal path instead.
__device__ __forceinline__ bool may_hit_exception(float s)
{
    const float h = 0.5f * s;
    const float t5 = 5.0f * h, t7 = 7.0f * h;                 // 10h shares t5's significand
    const uint32_t b5 = __float_as_uint(t5), b7 = __float_as_uint(t7);
    // a bf16 X with RN(X/h) = 5+ulp lies 0..4 binary32 steps above RN(5h); with RN(X/h) = 7-ulp,
    // 0..4 steps below RN(7h).  Zero steps only counts when the product was inexact.
    bool c5 = ((b5 + 4u) & 0xffffu) < 4u;
    bool c7 = ((b7 - 1u) & 0xffffu) < 4u;
    bool z5 = ((b5 & 0xffffu) == 0u) && (fmaf(5.0f, h, -t5) != 0.0f);
    bool z7 = ((b7 & 0xffffu) == 0u) && (fmaf(7.0f, h, -t7) != 0.0f);
    return c5 | c7 | z5 | z7;
}

__device__ __forceinline__ uint2 encode_rne_p32(const float (&v)[kBlock], float s)
{
    if (may_hit_exception(s) || near_threshold_hazard(s)) {   // ~1e-4 of blocks
        const float none[kBlock] = {};
        return encode_literal<0, false>(v, s, none);
    }
    const float rs = __builtin_amdgcn_rcpf(s);                // 1 ulp
    uint32_t lo = 0u, hi = 0u;
    // code = E2M1(x / s): x/s = (|x| / (s/2)) / 2 exactly, sign carried by the quotient
    lo = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(lo, div3(v[0], s, rs), div3(v[1], s, rs), 1.0f, 0);
    lo = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(lo, div3(v[2], s, rs), div3(v[3], s, rs), 1.0f, 1);
    lo = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(lo, div3(v[4], s, rs), div3(v[5], s, rs), 1.0f, 2);
    lo = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(lo, div3(v[6], s, rs), div3(v[7], s, rs), 1.0f, 3);
    hi = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(hi, div3(v[8], s, rs), div3(v[9], s, rs), 1.0f, 0);
    hi = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(hi, div3(v[10], s, rs), div3(v[11], s, rs), 1.0f, 1);
    hi = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(hi, div3(v[12], s, rs), div3(v[13], s, rs), 1.0f, 2);
    hi = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(hi, div3(v[14], s, rs), div3(v[15], s, rs), 1.0f, 3);
    return make_uint2(lo, hi);
}

// ---------------------------------------------------------------------------------------------
// Round-to-nearest, binary32 arithmetic on bf16 values, two operations per quotient.  The block scalar is a function
// of the block maximum alone, a bf16 value, so there are only 32 640 of them: quotient_table.h (written by
// gen_quotient_table.c, which walks every block maximum, every bf16 element below it and every reciprocal the
// hardware may return) has one bit per maximum that says whether
//     q = fma(x, rh, fma(x, rl, 0)),   rh = rcp(s),   rl = fma(-s, rh, 1) * rh        (rh + rl = 1/s to 2^-46)
// followed by the hardware conversion gives the reference's code for EVERY element such a block can hold.  All but 26
// maxima below 2^64 qualify; a block with any other maximum takes the literal sequence.  The inner fma adds +0 so that
// an input of -0.0 yields the quotient +0.0 (the reference's sign(-0.0) is 0).
// A workgroup stages the 4 KiB table in LDS once; N = 16 encodes a block, N = 8 one half of it (one packed word).
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ void stage_quotient_table(uint32_t* lds)      // every thread of the workgroup; ends with a barrier
{
    for (uint32_t i = threadIdx.x; i < (uint32_t)kQuotientTableWords / 4u; i += blockDim.x)
        reinterpret_cast<uint4*>(lds)[i] = reinterpret_cast<const uint4*>(kQuotientSafe)[i];
    __syncthreads();
}
__device__ __forceinline__ bool quotient_safe(const uint32_t* lds, float amax)   // amax >= 0, a bf16 value
{
    const uint32_t p = __float_as_uint(amax) >> 16;
    return ((lds[p >> 5] >> (p & 31u)) & 1u) != 0u;
}
struct SplitReciprocal { float hi, lo; };
__device__ __forceinline__ SplitReciprocal split_reciprocal(float s)
{
    SplitReciprocal r;
    r.hi = __builtin_amdgcn_rcpf(s);                          // 1 ulp
    r.lo = fmaf(-s, r.hi, 1.0f) * r.hi;
    return r;
}
__device__ __forceinline__ float quot2(float x, const SplitReciprocal r) { return fmaf(x, r.hi, fmaf(x, r.lo, 0.0f)); }

template <int N>
__device__ __forceinline__ void encode_p32_fast_n(const float (&v)[N], const SplitReciprocal r, uint32_t (&w)[N / 8])
{
#pragma unroll
    for (int k = 0; k < N / 8; ++k) {
        uint32_t c = 0u;
        // code = E2M1(x / s): x/s = (|x| / (s/2)) / 2 exactly, sign carried by the quotient
        c = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(c, quot2(v[8 * k], r), quot2(v[8 * k + 1], r), 1.0f, 0);
        c = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(c, quot2(v[8 * k + 2], r), quot2(v[8 * k + 3], r), 1.0f, 1);
        c = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(c, quot2(v[8 * k + 4], r), quot2(v[8 * k + 5], r), 1.0f, 2);
        c = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(c, quot2(v[8 * k + 6], r), quot2(v[8 * k + 7], r), 1.0f, 3);
        w[k] = c;
    }
}
template <int MODE, int N>
__device__ __forceinline__ void encode_literal_n(const float (&v)[N], float s, uint32_t (&w)[N / 8])
{
    const float h = rd<MODE>(s / 2.0f);
#pragma unroll
    for (int k = 0; k < N / 8; ++k) w[k] = 0u;
#pragma unroll
    for (int j = 0; j < N; ++j) {
        const float r = code_literal<MODE, false>(fabsf(v[j]), h, 0.0f);
        uint32_t code = (uint32_t)fminf(fmaxf(r, 0.0f), 7.0f);
        code |= (v[j] < 0.0f) ? 8u : 0u;
        w[j >> 3] |= code << (4 * (j & 7));
    }
}
// N elements of a block whose maximum is amax and whose scalar is s (binary32 arithmetic, bf16 values)
template <int N>
__device__ __forceinline__ void encode_rne_p32_tbl(const float (&v)[N], float amax, float s, const uint32_t* table, uint32_t (&w)[N / 8])
{
    if (quotient_safe(table, amax)) encode_p32_fast_n<N>(v, split_reciprocal(s), w);
    else encode_literal_n<0, N>(v, s, w);
}

// Round-to-nearest, binary32 arithmetic, on binary32 VALUES (inputs that are not bf16 values: a binary32
// tensor, or a bf16 tensor minus a binary32 centre).  The block-level guards of encode_rne_p32 reason about
// bf16 inputs and do not apply; here every quotient is tested instead.  div3 is a faithful quotient for any
// binary32 x (its remainder step is exact), so it is within 1 ulp of RN(x/s); the reference's code can differ
// from the round-to-nearest-even conversion of div3 only if a decision threshold, or one of the three
// exceptional quotients next to 2.5, 3.5 and 5, lies within that distance.  Every threshold has zero low 20
// significand bits, so a quotient whose low 20 bits are within 4 of 0 (mod 2^20) sends the block to the literal
// sequence: about 1e-4 of blocks.  Quotients below 0.125 encode as 0 and quotients above 5.5 as 7 either way and
// are never flagged (zeros are common, and every block's maximum has a quotient just below 6).  Checked on the host against the literal sequence on 9e8 cases around every threshold.
__device__ __forceinline__ uint2 encode_rne_wide(const float (&v)[kBlock], float s)
{
    const float rs = __builtin_amdgcn_rcpf(s);                // 1 ulp
    // the quotients are converted as they are formed (nothing but the two packed words stays live); the rare
    // flagged block is redone literally afterwards
    // all in vector integer ops (no compares): magnitudes outside [0.125, 5.5] are clamped to patterns that never flag,
    // bits 3..19 of (pattern + 4) are zero exactly for a flagged quotient, and the minimum over the block is kept
    uint32_t lo = 0u, hi = 0u, least = 0xffffffffu;
    auto quot = [&](int j) {
        const float q = div3(v[j], s, rs);
        uint32_t a = __float_as_uint(q) & 0x7fffffffu;
        a = a < 0x3e000010u ? 0x3e000010u : a;                 // below 0.125: code 0 either way
        a = a > 0x40b00010u ? 0x40b00010u : a;                 // above 5.5: code 7 (every block maximum sits at 6)
        const uint32_t m = ((a + 4u) >> 3) & 0x1ffffu;
        least = m < least ? m : least;
        return q;
    };
    lo = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(lo, quot(0), quot(1), 1.0f, 0);
    lo = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(lo, quot(2), quot(3), 1.0f, 1);
    lo = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(lo, quot(4), quot(5), 1.0f, 2);
    lo = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(lo, quot(6), quot(7), 1.0f, 3);
    hi = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(hi, quot(8), quot(9), 1.0f, 0);
    hi = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(hi, quot(10), quot(11), 1.0f, 1);
    hi = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(hi, quot(12), quot(13), 1.0f, 2);
    hi = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(hi, quot(14), quot(15), 1.0f, 3);
    const bool flagged = least == 0u;
    if (__builtin_amdgcn_ballot_w64(flagged) != 0ull) {        // wave-uniform: a real branch around the long sequence
        // Element by element: the literal rule only for the positions at which some lane of the wave holds a flagged
        // quotient (tensors with short mantissas flag a few quotients in most waves: redoing whole blocks cost 40 %).
        const float h = rd<0>(s / 2.0f);
        uint32_t w[2] = {lo, hi};
#pragma unroll
        for (int j = 0; j < kBlock; ++j) {
            const float q = div3(v[j], s, rs);
            uint32_t a = __float_as_uint(q) & 0x7fffffffu;
            a = a < 0x3e000010u ? 0x3e000010u : a;
            a = a > 0x40b00010u ? 0x40b00010u : a;
            const bool fj = (((a + 4u) >> 3) & 0x1ffffu) == 0u;
            if (__builtin_amdgcn_ballot_w64(fj) != 0ull) {
                const float r = code_literal<0, false>(fabsf(v[j]), h, 0.0f);
                uint32_t code = (uint32_t)fminf(fmaxf(r, 0.0f), 7.0f);
                code |= (v[j] < 0.0f) ? 8u : 0u;
                const uint32_t sh = 4u * (uint32_t)(j & 7);
                if (fj) w[j >> 3] = (w[j >> 3] & ~(0xFu << sh)) | (code << sh);
            }
        }
        lo = w[0];
        hi = w[1];
    }
    return make_uint2(lo, hi);
}

// Round-to-nearest, every op rounded to bf16.  With q = bf16(RN(|x| / h)) the reference's
// compress/round/expand sequence is a function of the bf16 value q alone, and over all bf16 q in
// [0, 13] it equals the round-to-nearest-even conversion onto the E2M1 grid except at q = 5+1ulp,
// 7-1ulp and 10+1ulp (bf16 ulps), where its intermediate roundings land on the tie 5, 7, 10.
// div3() followed by the bf16 rounding gives exactly bf16(RN(x / h)) for bf16 x and h: a binary32
// quotient that is not exactly representable stays at least 2^-17 (relative) away from every bf16
// midpoint, far more than div3's error.  Checked on the host for every (h, x) pair of bf16 values.
__device__ __forceinline__ float nudge_pb16(float q)          // q >= 0
{
    q = (q == 5.03125f) ? 5.0f : q;
    q = (q == 6.96875f) ? 7.0f : q;
    q = (q == 10.0625f) ? 10.0f : q;
    return q;
}
__device__ __forceinline__ uint2 encode_rne_pb16(const float (&v)[kBlock], float s)
{
    const float h = 0.5f * s;                                 // bf16(s / 2), exact
    const float rh = __builtin_amdgcn_rcpf(h);                // 1 ulp
    uint32_t w[2] = {0u, 0u}, sg[2] = {0u, 0u};
#pragma unroll
    for (int j = 0; j < kBlock; j += 2) {
        // signed quotients: div3 turns a -0.0 input into +0.0, which is the reference's sign(x) = 0
        const uint32_t qq = rb_pair(div3(v[j], h, rh), div3(v[j + 1], h, rh));
        const float q0 = nudge_pb16(fabsf(bf16_lo(qq))), q1 = nudge_pb16(fabsf(bf16_hi(qq)));
        sg[j >> 3] |= (((qq >> 12) & 0x8u) | ((qq >> 24) & 0x80u)) << (4 * (j & 7));
        // magnitude code = E2M1(q / 2): the converter divides by the power of two given as its scale
        switch ((j >> 1) & 3) {
        case 0: w[j >> 3] = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w[j >> 3], q0, q1, 2.0f, 0); break;
        case 1: w[j >> 3] = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w[j >> 3], q0, q1, 2.0f, 1); break;
        case 2: w[j >> 3] = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w[j >> 3], q0, q1, 2.0f, 2); break;
        default: w[j >> 3] = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w[j >> 3], q0, q1, 2.0f, 3); break;
        }
    }
    return make_uint2(w[0] | sg[0], w[1] | sg[1]);
}

// the same for N elements (8: half a block, one packed word)
template <int N>
__device__ __forceinline__ void encode_rne_pb16_n(const float (&v)[N], float s, uint32_t (&out)[N / 8])
{
    const float h = 0.5f * s;
    const float rh = __builtin_amdgcn_rcpf(h);
#pragma unroll
    for (int k = 0; k < N / 8; ++k) {
        uint32_t w = 0u, sg = 0u;
#pragma unroll
        for (int j = 0; j < 8; j += 2) {
            const uint32_t qq = rb_pair(div3(v[8 * k + j], h, rh), div3(v[8 * k + j + 1], h, rh));
            const float q0 = nudge_pb16(fabsf(bf16_lo(qq))), q1 = nudge_pb16(fabsf(bf16_hi(qq)));
            sg |= (((qq >> 12) & 0x8u) | ((qq >> 24) & 0x80u)) << (4 * j);
            switch (j >> 1) {
            case 0: w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, q0, q1, 2.0f, 0); break;
            case 1: w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, q0, q1, 2.0f, 1); break;
            case 2: w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, q0, q1, 2.0f, 2); break;
            default: w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, q0, q1, 2.0f, 3); break;
            }
        }
        out[k] = w | sg;
    }
}

// One v_cvt_scalef32_sr_pk_fp4_f32: converts (q0, q1) / 2^MODE with stochastic rounding into byte `byte` of w
// and keeps w's other bytes.  Written as assembly because the compiler builtin of this ROCm release does not
// tie the previous value of the destination to the instruction (the other bytes came back undefined); the
// leading s_nop covers the wait state a partial (op_sel) write needs before the register is read again.
template <int MODE>
__device__ __forceinline__ void sr_convert_pair(uint32_t& w, float q0, float q1, uint32_t bits, int byte)
{
    typedef float pair_t __attribute__((ext_vector_type(2)));
    const pair_t q = {q0, q1};
#define METIS_SR_CVT(SCALE, SEL) asm("s_nop 0\n\tv_cvt_scalef32_sr_pk_fp4_f32 %0, %1, %2, " SCALE SEL : "+v"(w) : "v"(q), "v"(bits))
    if (MODE == 0) {
        if (byte == 0) METIS_SR_CVT("1.0", "");
        else if (byte == 1) METIS_SR_CVT("1.0", " op_sel:[0,0,1,0]");
        else if (byte == 2) METIS_SR_CVT("1.0", " op_sel:[0,0,0,1]");
        else METIS_SR_CVT("1.0", " op_sel:[0,0,1,1]");
    } else {
        if (byte == 0) METIS_SR_CVT("2.0", "");
        else if (byte == 1) METIS_SR_CVT("2.0", " op_sel:[0,0,1,0]");
        else if (byte == 2) METIS_SR_CVT("2.0", " op_sel:[0,0,0,1]");
        else METIS_SR_CVT("2.0", " op_sel:[0,0,1,1]");
    }
#undef METIS_SR_CVT
}

// Stochastic rounding with the library's own random stream.  The reference adds U(-1/2, 1/2) to the
// compressed quotient and rounds to nearest (src/Metis/Metis/quant.py:137-147); compress is linear
// between neighbouring grid points, so this is plain stochastic rounding onto the E2M1 grid:
// P(up) = (q - lo) / (hi - lo).  The hardware converter v_cvt_scalef32_sr_pk_fp4_f32 does exactly
// that from 32 random bits per element pair (measured on hardware: unbiased over 2^20 seeds for
// every grid interval, saturating at 6, sign kept, the two elements of a pair read the random
// word one bit apart).  One Philox4x32-10 draw serves a block: counter = offset + output block,
// pair p (elements 2p, 2p+1) takes word p % 4, rotated by 16 bits for p >= 4 (the converter only
// looks at the top 13 bits).  Scale bytes and unit do not depend on the rounding mode.
// WIDE_VALUES: the input need not be bf16-valued, which div3's exactness argument assumes; the quotient is then
// x * rcp(s), within 2 ulp of x / s.  Stochastic rounding does not need more: the probability of rounding up
// moves by 1e-7 of a grid interval, and a quotient that lands above 6 saturates in the converter either way.
template <int MODE, bool WIDE_VALUES = false>
__device__ __forceinline__ uint2 encode_sr_hardware(const float (&v)[kBlock], float s, uint64_t seed, uint64_t offset,
                                                    int64_t ob)
{
    const uint4 r = Philox::draw(offset + (uint64_t)ob, seed);
    const uint32_t word[4] = {r.x, r.y, r.z, r.w};
    // MODE 0: x / s in binary32 (div3 is a faithful rounding of the quotient).  MODE 1: bf16(x / h), h = s / 2.
    const float d = MODE ? 0.5f * s : s;
    const float rd_ = __builtin_amdgcn_rcpf(d);
    uint32_t w[2] = {0u, 0u};
#pragma unroll
    for (int j = 0; j < kBlock; j += 2) {
        const int p = j >> 1;
        const uint32_t bits = p < 4 ? word[p] : __builtin_amdgcn_alignbit(word[p & 3], word[p & 3], 16);
        // "+ 0.0f" turns a -0.0 quotient into +0.0, as div3 does: the reference's sign(x) is 0 for x = -0.0
        float q0 = WIDE_VALUES ? v[j] * rd_ + 0.0f : div3(v[j], d, rd_);
        float q1 = WIDE_VALUES ? v[j + 1] * rd_ + 0.0f : div3(v[j + 1], d, rd_);
        if (MODE) {
            const uint32_t qq = rb_pair(q0, q1);
            q0 = bf16_lo(qq);
            q1 = bf16_hi(qq);
        }
        sr_convert_pair<MODE>(w[p >> 2], q0, q1, bits, p & 3);
    }
    return make_uint2(w[0], w[1]);
}

template <int MODE, bool SR>
__device__ __forceinline__ uint2 encode_block(const float (&v)[kBlock], float s, const float (&u)[kBlock])
{
    if constexpr (MODE == 0 && !SR) return encode_rne_p32(v, s);
    else if constexpr (MODE == 1 && !SR) return encode_rne_pb16(v, s);
    else return encode_literal<MODE, SR>(v, s, u);
}

__device__ __forceinline__ float block_amax(const float (&v)[kBlock])
{
    float m = 0.0f;
#pragma unroll
    for (int j = 0; j < kBlock; j += 2) m = amax3(m, v[j], v[j + 1]);
    return m;
}

// maximum magnitude of the 16 packed bf16 values, computed on the bit patterns (two per dword)
typedef unsigned short ushort2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float block_amax_packed(const uint4 a, const uint4 b)
{
    const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    ushort2_t m[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) m[j] = __builtin_bit_cast(ushort2_t, w[j] & 0x7fff7fffu);
#pragma unroll
    for (int j = 0; j < 4; ++j) m[j] = __builtin_elementwise_max(m[j], m[j + 4]);
    m[0] = __builtin_elementwise_max(__builtin_elementwise_max(m[0], m[1]), __builtin_elementwise_max(m[2], m[3]));
    const uint32_t r = __builtin_bit_cast(uint32_t, m[0]);
    const uint32_t hi = r >> 16, lo = r & 0xffffu;
    return __uint_as_float((hi > lo ? hi : lo) << 16);
}

__device__ __forceinline__ void unpack16(const uint4 a, const uint4 b, float (&v)[kBlock])
{
    const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) { v[2 * j] = bf16_lo(w[j]); v[2 * j + 1] = bf16_hi(w[j]); }
}

// Tiled random Hadamard rotation of the NV recipe on one tile of 16 in registers (the tile is the scale block).
// Forward: (v * sign) H, src/Metis/Metis/bitlinear.py:199-202; inverse: (v H) / 16 * sign, bitlinear.py:195-197, with H the
// Sylvester matrix (75-96) and sign the shared vector of 126-137, here a bit mask (bit j set: sign[j] = -1).
// The reference forms v H as a binary32 matrix product (torch.mm on the CPU): every output is the sum of its sixteen
// terms +-v[k] taken in the order k = 0 .. 15.  The order matters: the weight gradient's second operand is the already
// quantized input rotated and quantized AGAIN, its rotated values sit on FP4 rounding boundaries far more often than
// ordinary data, and which side they land on hangs on the last bit of these sums.  Summed in this order the kernels
// reproduce the reference's operand bit for bit (a butterfly network, or a double-precision sum rounded once, each
// leave 5 % of that operand's elements different: 2e-2 in the Frobenius norm).  240 additions instead of the
// network's 64; H[k][n] = (-1)^popcount(k & n) is folded at compile time.
__device__ __forceinline__ void hadamard16_product(float (&v)[kBlock])
{
    float o[kBlock];
#pragma unroll
    for (int n = 0; n < kBlock; ++n) {
        float acc = v[0];                                     // H[0][n] = +1, and 0 + v[0] = v[0]
#pragma unroll
        for (int k = 1; k < kBlock; ++k) acc = (__builtin_popcount(k & n) & 1) ? acc - v[k] : acc + v[k];
        o[n] = acc;
    }
#pragma unroll
    for (int n = 0; n < kBlock; ++n) v[n] = o[n];
}
__device__ __forceinline__ void hadamard16_forward(float (&v)[kBlock], uint32_t sign_mask)
{
#pragma unroll
    for (int j = 0; j < kBlock; ++j) v[j] = __uint_as_float(__float_as_uint(v[j]) ^ (((sign_mask >> j) & 1u) << 31));
    hadamard16_product(v);
}
__device__ __forceinline__ void hadamard16_inverse(float (&v)[kBlock], uint32_t sign_mask)
{
    hadamard16_product(v);
#pragma unroll
    for (int j = 0; j < kBlock; ++j) v[j] = __uint_as_float(__float_as_uint(v[j] * 0.0625f) ^ (((sign_mask >> j) & 1u) << 31));
}

// publish the workgroup's maximum block-maximum (non-negative floats order like their bit patterns).
// fill_to: entries gridDim.x .. fill_to-1 are cleared as well, for readers that always fold a fixed number of entries.
// (block, grid: the workgroup's index among the `grid` workgroups that publish, when that is not the whole launch)
__device__ __forceinline__ void publish_group_max(float m, uint32_t* ws_gmax, uint32_t fill_to, uint32_t block, uint32_t grid)
{
    __shared__ float smax[4];
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) smax[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) ws_gmax[block] = __float_as_uint(fmaxf(fmaxf(smax[0], smax[1]), fmaxf(smax[2], smax[3])));
    for (uint32_t j = grid + block * 256u + threadIdx.x; j < fill_to; j += grid * 256u) ws_gmax[j] = 0u;
}
__device__ __forceinline__ void publish_group_max(float m, uint32_t* ws_gmax, uint32_t fill_to = 0)
{
    publish_group_max(m, ws_gmax, fill_to, blockIdx.x, gridDim.x);
}

// Deferred scale bytes: a quantizer call may stop after phase 1 and hand its parked bf16 block maxima and its partial
// maxima (always kDeferredPartials entries, unused ones zero) to the consumer, which forms the tensor unit and the E4M3
// bytes itself (quant.py:21-23) -- the same expressions as quant_scales_kernel, so the same bits.
constexpr uint32_t kDeferredPartials = 2048;
// tensor maximum from the partial maxima: every thread of a 256-thread workgroup calls this
__device__ __forceinline__ float fold_partial_maxima(const uint32_t* __restrict__ partials)
{
    static_assert(kDeferredPartials == 256 * 8, "256 threads fold eight entries each");
    __shared__ float fmax_s[4];
    const uint4 a = reinterpret_cast<const uint4*>(partials)[threadIdx.x];
    const uint4 b = reinterpret_cast<const uint4*>(partials)[threadIdx.x + 256];
    float m = fmaxf(fmaxf(fmaxf(__uint_as_float(a.x), __uint_as_float(a.y)), fmaxf(__uint_as_float(a.z), __uint_as_float(a.w))),
                    fmaxf(fmaxf(__uint_as_float(b.x), __uint_as_float(b.y)), fmaxf(__uint_as_float(b.z), __uint_as_float(b.w))));
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) fmax_s[threadIdx.x >> 6] = m;
    __syncthreads();
    return fmaxf(fmaxf(fmax_s[0], fmax_s[1]), fmaxf(fmax_s[2], fmax_s[3]));
}
template <int MODE>
__device__ __forceinline__ float tensor_unit_of(float amax) { return rd<MODE>(block_scalar<MODE>(amax) / 448.0f); }
template <int MODE>
__device__ __forceinline__ uint32_t scale_byte_of(uint32_t amax_bf16, float unit)
{
    return e4m3_byte(rd<MODE>(block_scalar<MODE>(__uint_as_float(amax_bf16 << 16)) / unit));
}

}  // namespace metis
