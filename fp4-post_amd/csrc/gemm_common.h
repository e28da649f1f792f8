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

}  // namespace metis
