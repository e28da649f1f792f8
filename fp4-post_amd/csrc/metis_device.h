// Device-side helpers shared by the Metis NVFP4 kernels (gfx950 only).
//
// Arithmetic contract: everything that decides a stored bit (E2M1 code, E4M3 scale byte, unit)
// reproduces the reference's eager op sequence on CPU (src/Metis/Metis/quant.py:6-36): IEEE
// binary32 operations in that order, true divisions, and -- in bf16-per-op mode -- a round to
// bf16 after every operation.  The file is compiled with -ffp-contract=off; fused multiply-adds
// appear only where written explicitly.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace metis {

constexpr int kBlock = 16;            // elements per scale block (quant.py:181 block_shape)
constexpr int kMaxGroups = 4096;      // upper bound on workgroups that publish a partial maximum

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// binary32 -> bf16 round-to-nearest-even (hardware convert), result widened back to binary32.
__device__ __forceinline__ uint32_t bf16_bits(float f)
{
    return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f);
}
__device__ __forceinline__ float rb(float f) { return __uint_as_float(bf16_bits(f) << 16); }
// two roundings to bf16 at once, packed (first argument in the low half): one v_cvt_pk_bf16_f32
typedef float metis_float2_t __attribute__((ext_vector_type(2)));
typedef __bf16 metis_bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t rb_pair(float lo, float hi)
{
    const metis_float2_t f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, metis_bf16x2_t));
}
template <int MODE> __device__ __forceinline__ float rd(float v) { return MODE ? rb(v) : v; }

// a / 6 correctly rounded for every bf16-valued a (exhaustively checked on the host):
// constant reciprocal, exact remainder, one correction.
__device__ __forceinline__ float div6(float a)
{
    const float c = 0x1.555556p-3f;   // RN(1/6)
    float q = a * c;
    float r = fmaf(-6.0f, q, a);
    return fmaf(r, c, q);
}

// quant.py:19  scalar = amax / 6 + 1e-9   (each op rounded to bf16 in mode 1)
template <int MODE> __device__ __forceinline__ float block_scalar(float amax)
{
    return rd<MODE>(rd<MODE>(div6(amax)) + 1e-9f);
}

// x / s for a bf16-valued x (8 significant bits), given rs within 1 ulp of 1/s: product, exact
// remainder, one correction.  Before its final rounding the value is within 2^-44 (relative) of
// x/s, so the result is a faithful rounding of x/s and is RN(x/s) whenever x/s is exactly
// representable (all exact ties).  It can differ from RN(x/s) only when x/s lies within 2^-44 of
// a midpoint between two binary32 numbers; near an E2M1 decision threshold W (k/4, k in
// {1,3,5,7,10,14,20}) that requires the low 20 bits of the significand of s to be a non-zero
// value within 64 of 0 modulo 2^20 -- see near_threshold_hazard() -- because x - W*s is a multiple
// of ulp(s)/4 while the half-ulp offset of the midpoint is s * 2^(E_W-24).
__device__ __forceinline__ float div3(float x, float s, float rs)
{
    float w = x * rs;
    float e = fmaf(-s, w, x);
    return fmaf(e, rs, w);
}
__device__ __forceinline__ bool near_threshold_hazard(float s)
{
    const uint32_t t = __float_as_uint(s) & 0xfffffu;
    return (t != 0u) & (((t + 64u) & 0xfffffu) <= 128u);
}

// max(acc, |a|, |b|) in one instruction, without the NaN canonicalisation that fmaxf adds
__device__ __forceinline__ float amax3(float acc, float a, float b)
{
    float r;
    asm("v_max3_f32 %0, %1, |%2|, |%3|" : "=v"(r) : "v"(acc), "v"(a), "v"(b));
    return r;
}

// float8_e4m3fn byte of a non-negative binary32 value (round to nearest even; > 464 -> 0x7F).
// The gfx950 converter implements the OCP format and agrees with PyTorch's cast on every
// byte boundary, midpoint and neighbour (checked on hardware).
__device__ __forceinline__ uint32_t e4m3_byte(float t)
{
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(t, 0.0f, 0, false) & 0xffu;
}
__device__ __forceinline__ float e4m3_value(uint32_t b)   // finite bytes
{
    uint32_t e = (b >> 3) & 15u, m = b & 7u;
    float mag = e ? __uint_as_float(((e + 120u) << 23) | (m << 20)) : (float)m * 0x1p-9f;
    return (b & 0x80u) ? -mag : mag;
}

// quant.py:27-31 literally, for one element: |x| / h, compress, (noise), round half to even.
// h = scalar / 2.  Returns the rounded compressed magnitude (0..8).
template <int MODE, bool SR>
__device__ __forceinline__ float code_literal(float ax, float h, float u)
{
    float q = rd<MODE>(ax / h);
    float t1 = rd<MODE>(fmaxf(rd<MODE>(q - 4.0f), 0.0f) / 2.0f);
    float t2 = rd<MODE>(fmaxf(rd<MODE>(q - 8.0f), 0.0f) / 4.0f);
    float c = rd<MODE>(q - rd<MODE>(t1 + t2));
    if (SR) c = rd<MODE>(c + rd<MODE>(u - 0.5f));
    return rintf(c);
}

// Philox4x32-10 (Salmon et al., SC'11): counter-based generator for stochastic rounding.
struct Philox {
    static __device__ __forceinline__ uint4 draw(uint64_t ctr, uint64_t seed)
    {
        uint32_t c0 = (uint32_t)ctr, c1 = (uint32_t)(ctr >> 32), c2 = 0u, c3 = 0u;
        uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
#pragma unroll
        for (int i = 0; i < 10; ++i) {
            // both halves of each product from one 32 x 32 -> 64 bit multiply-add (integer multiplies run at quarter rate)
            const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
            const uint32_t h0 = (uint32_t)(p0 >> 32), l0 = (uint32_t)p0, h1 = (uint32_t)(p1 >> 32), l1 = (uint32_t)p1;
            c0 = h1 ^ c1 ^ k0; c1 = l1; c2 = h0 ^ c3 ^ k1; c3 = l0;
            k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
        }
        return make_uint4(c0, c1, c2, c3);
    }
};
// uniform in [0,1) with the granularity torch.rand uses for the dtype: 2^-24 (float32), 2^-8 (bf16)
template <int MODE> __device__ __forceinline__ float uniform_from_bits(uint32_t r)
{
    return MODE ? (float)(r >> 24) * 0x1p-8f : (float)(r >> 8) * 0x1p-24f;
}

// wave-wide maximum of non-negative floats (64 lanes)
__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

}  // namespace metis
