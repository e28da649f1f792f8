/*
 * Plain-C restatement of the Metis NVFP4 quantizer arithmetic (TEST INFRASTRUCTURE).
 *
 * This file is a checker and a CPU baseline, never a product path: only the tests, the
 * smoke check and the benchmark's CPU-baseline leg load the library built from it.
 *
 * It restates the reference's op sequence with scalar IEEE-754 binary32 operations
 * (compile with -ffp-contract=off, no fast-math) and an explicit round-to-bf16 after each
 * operation in mode 1, which is what eager PyTorch does on a bf16 tensor (compute in float,
 * store bf16).  Python scalars (6, 1e-9, 448, 2, 4, 8, 0.5) enter as binary32 values.
 *
 * Reference files followed:
 *   src/Metis/Metis/quant.py:6-36      fused NVFP4 QDQ (RNE)
 *   src/Metis/Metis/quant.py:118-128   E2M1 compress / round / expand
 *   src/Metis/Metis/quant.py:137-147   stochastic rounding: += rand - 0.5 before round
 *   src/Metis/Metis/quant.py:435-477   get_scalar / quant / rquant
 *   src/Metis/models/llama.py:23-31    RMSNorm
 *   src/Metis/Metis/bitlinear.py:296   ker = ug @ diag(sg) @ vg, with the summation order FIXED here (see
 *                                      metis_oracle_lowrank_product; the reference leaves it to its BLAS)
 * Third-party arithmetic restated from its published definition (absent from the reference
 * tree): the float8_e4m3fn cast of PyTorch (OCP FP8 E4M3: bias 7, 3 mantissa bits, no
 * infinities, 0x7F/0xFF = NaN, round-to-nearest-even, values that round above 448 -> NaN).
 *
 * mode 0 (P32) : binary32 arithmetic on the bf16-valued inputs
 * mode 1 (PB16): every operation rounded to bf16
 */
#include <math.h>
#include <stdint.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define BLK 16

static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bf16_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* binary32 -> bf16, round to nearest even; NaN stays a quiet NaN */
uint16_t metis_oracle_f32_to_bf16(float f)
{
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t keep_odd = (u >> 16) & 1u;
    return (uint16_t)((u + 0x7fffu + keep_odd) >> 16);
}
static inline float rb(float f) { return bf16_f32(metis_oracle_f32_to_bf16(f)); }
/* RD(mode, v): value after the store of one eager op */
#define RD(mode, v) ((mode) ? rb(v) : (v))

/* float8_e4m3fn value of a byte */
float metis_oracle_e4m3_decode(uint8_t b)
{
    int e = (b >> 3) & 0xF, m = b & 7;
    float mag;
    if (e == 15 && m == 7) mag = NAN;
    else if (e == 0) mag = ldexpf((float)m, -9);             /* subnormal: m * 2^-9 */
    else mag = ldexpf(1.0f + (float)m / 8.0f, e - 7);
    return (b & 0x80) ? -mag : mag;
}

/* binary32 -> float8_e4m3fn byte, round to nearest even */
uint8_t metis_oracle_e4m3_encode(float f)
{
    uint8_t sign = (uint8_t)((f32_bits(f) >> 24) & 0x80u);
    float a = fabsf(f);
    if (!(a == a)) return sign | 0x7F;
    if (a >= 480.0f) return sign | 0x7F;                      /* beyond the last rounding interval */
    if (a < 0.015625f) {                                      /* below 2^-6: multiples of 2^-9 */
        int n = (int)rintf(a * 512.0f);                       /* exact scaling, RNE */
        return sign | (uint8_t)n;                             /* n == 8 is the first normal */
    }
    int ex;
    float fr = frexpf(a, &ex);                                /* a = fr * 2^ex, fr in [0.5,1) */
    int k = (int)rintf(fr * 16.0f);                           /* 4 significant bits, RNE */
    if (k == 16) { k = 8; ex += 1; }
    int field = ex - 1 + 7;
    int byte = (field << 3) | (k - 8);
    if (byte >= 0x7F) return sign | 0x7F;                     /* [464,480) rounds up past 448 */
    return sign | (uint8_t)byte;
}

static inline float relu(float v) { return v > 0.0f ? v : 0.0f; }

/* quant.py:27-31 (+144-145): rounded compressed magnitude for one element.
 * h = scalar/2; use_noise = 0 selects round-to-nearest (no noise term). */
static inline float element_code(float ax, float h, int mode, int use_noise, float u)
{
    float q  = RD(mode, ax / h);
    float t1 = RD(mode, relu(RD(mode, q - 4.0f)) / 2.0f);
    float t2 = RD(mode, relu(RD(mode, q - 8.0f)) / 4.0f);
    float c  = RD(mode, q - RD(mode, t1 + t2));
    if (use_noise) c = RD(mode, c + RD(mode, u - 0.5f));
    return rintf(c);                                          /* torch.round: half to even */
}

static const float k_twice[8] = {0.f, 1.f, 2.f, 3.f, 4.f, 6.f, 8.f, 12.f};

/* quant.py:19: raw block scalar from the block maximum */
static inline float block_scalar(float amax, int mode)
{
    return RD(mode, RD(mode, amax / 6.0f) + 1e-9f);
}

/*
 * Pack a [rows, cols] bf16 tensor (binary32 in mode 2; row stride ld elements) into NVFP4.
 *   codes  [rows, cols/2]  element 2j in the low nibble of byte j; nibble = (x<0)<<3 | r
 *   scales [rows, cols/16] float8_e4m3fn byte of scalar/unit
 *   unit   = max(scalar)/448 (bf16-valued in mode 1)
 *   noise  NULL for RNE; else uniform draws in [0,1): float32[rows*cols] in mode 0,
 *          bf16 bits uint16[rows*cols] in mode 1
 *   n_clamped (optional) counts SR elements whose r rounded to 8 and were clamped to 7
 * Returns 0, or -1 when 16 does not divide cols.
 */
int metis_oracle_nvfp4_pack(const void *xin, int64_t rows, int64_t cols, int64_t ld, int mode,
                            const void *noise, uint8_t *codes, uint8_t *scales, float *unit,
                            int64_t *n_clamped)
{
    /* mode 2: the arithmetic of mode 0 on a binary32 tensor (the reference run with compute_dtype=float32 on
     * values that are not bf16 values, e.g. gradients: bitlinear.py:453) */
    const int f32in = mode == 2;
    if (f32in) mode = 0;
    const uint16_t *x = (const uint16_t *)xin;
    const float *xf = (const float *)xin;
#define LDX(i) (f32in ? xf[i] : bf16_f32(x[i]))
    if (cols % BLK) return -1;
    const int64_t nb = cols / BLK;
    float smax = 0.0f;
    /* pass 1: tensor maximum of the raw scalars (quant.py:21) */
#pragma omp parallel for reduction(max : smax) schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        for (int64_t b = 0; b < nb; ++b) {
            float am = 0.0f;
            for (int j = 0; j < BLK; ++j) {
                float a = fabsf(LDX(r * ld + b * BLK + j));
                am = a > am ? a : am;
            }
            float s = fabsf(block_scalar(am, mode));
            smax = s > smax ? s : smax;
        }
    }
    const float un = RD(mode, smax / 448.0f);                 /* quant.py:22 */
    *unit = un;
    int64_t clamped = 0;
#pragma omp parallel for reduction(+ : clamped) schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        for (int64_t b = 0; b < nb; ++b) {
            const int64_t xb = r * ld + b * BLK;
            float am = 0.0f;
            for (int j = 0; j < BLK; ++j) {
                float a = fabsf(LDX(xb + j));
                am = a > am ? a : am;
            }
            const float s = block_scalar(am, mode);
            scales[r * nb + b] = metis_oracle_e4m3_encode(RD(mode, s / un));   /* quant.py:23 */
            const float h = RD(mode, s / 2.0f);
            uint8_t nib[BLK];
            for (int j = 0; j < BLK; ++j) {
                float xv = LDX(xb + j);
                float u = 0.0f;
                if (noise) {
                    int64_t idx = r * cols + b * BLK + j;
                    u = mode ? bf16_f32(((const uint16_t *)noise)[idx]) : ((const float *)noise)[idx];
                }
                float rr = element_code(fabsf(xv), h, mode, noise != NULL, u);
                int code = (int)rr;
                if (code > 7) { code = 7; ++clamped; }
                if (code < 0) code = 0;
                nib[j] = (uint8_t)(code | ((xv < 0.0f) ? 8 : 0));
            }
            for (int j = 0; j < BLK / 2; ++j)
                codes[r * (cols / 2) + b * (BLK / 2) + j] = (uint8_t)(nib[2 * j] | (nib[2 * j + 1] << 4));
        }
    }
    if (n_clamped) *n_clamped = clamped;
    return 0;
#undef LDX
}

/*
 * Dequantize: quant.py:23-24 and 32-35 applied to the stored integers,
 *   out = ((v * sign) / 2) * (e4m3 * unit)   with the per-op rounding of the mode.
 * out_bf16 / out_f32 may each be NULL.  In mode 0 the bf16 output is the final value rounded
 * once to bf16; in mode 1 the value is already bf16.
 */
int metis_oracle_nvfp4_dequant(const uint8_t *codes, const uint8_t *scales, float unit, int64_t rows,
                               int64_t cols, int mode, uint16_t *out_bf16, float *out_f32)
{
    if (cols % BLK) return -1;
    const int64_t nb = cols / BLK;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        for (int64_t b = 0; b < nb; ++b) {
            float dq = RD(mode, metis_oracle_e4m3_decode(scales[r * nb + b]) * unit);
            for (int j = 0; j < BLK; ++j) {
                uint8_t byte = codes[r * (cols / 2) + (b * BLK + j) / 2];
                uint8_t nb4 = (j & 1) ? (byte >> 4) : (byte & 0xF);
                float v = k_twice[nb4 & 7];
                float sg = (nb4 & 8) ? -1.0f : 1.0f;
                float val = RD(mode, RD(mode, RD(mode, v * sg) / 2.0f) * dq);
                int64_t o = r * cols + b * BLK + j;
                if (out_f32) out_f32[o] = val;
                if (out_bf16) out_bf16[o] = metis_oracle_f32_to_bf16(val);
            }
        }
    }
    return 0;
}

/*
 * RMSNorm, llama.py:23-31 with a bf16 weight: binary32 x * rsqrt(mean(x^2) + eps), rounded to
 * bf16, times gamma, rounded to bf16.  The mean is accumulated in double (PyTorch's own
 * summation order is not part of the contract; results agree to rounding of the mean).
 */
int metis_oracle_rmsnorm(const uint16_t *x, const uint16_t *gamma, float eps, int64_t rows,
                         int64_t cols, uint16_t *out)
{
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        double acc = 0.0;
        for (int64_t c = 0; c < cols; ++c) {
            float v = bf16_f32(x[r * cols + c]);
            acc += (double)(v * v);
        }
        float mean = (float)(acc / (double)cols);
        float rstd = 1.0f / sqrtf(mean + eps);
        for (int64_t c = 0; c < cols; ++c) {
            float n = rb(bf16_f32(x[r * cols + c]) * rstd);
            out[r * cols + c] = metis_oracle_f32_to_bf16(n * bf16_f32(gamma[c]));
        }
    }
    return 0;
}

/* RMSNorm followed by NVFP4 packing of the normed tensor (contract of the fused kernel). */
int metis_oracle_rmsnorm_nvfp4(const uint16_t *x, const uint16_t *gamma, float eps, int64_t rows,
                               int64_t cols, int mode, uint16_t *normed, uint8_t *codes,
                               uint8_t *scales, float *unit)
{
    if (cols % BLK) return -1;
    metis_oracle_rmsnorm(x, gamma, eps, rows, cols, normed);
    return metis_oracle_nvfp4_pack(normed, rows, cols, cols, mode, NULL, codes, scales, unit, NULL);
}

/*
 * ker = us @ vt (src/Metis/Metis/bitlinear.py:296 after `ug @ torch.diag(sg)`), binary32, [rows, rank] x [rank, cols].
 * The reference calls a library matrix product, whose order of additions is the library's own.  This restatement fixes
 * one: acc = 0; acc = fma(us[i][k], vt[k][j], acc) for k = 0 .. rank-1.  It is the order the HIP kernel uses, so the two
 * agree bit for bit; against the reference's product it agrees to rounding (checked on the reference's own vectors).
 */
int metis_oracle_lowrank_product(const float *us, const float *vt, int64_t rows, int64_t cols, int64_t rank, float *ker)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows; ++i)
        for (int64_t j = 0; j < cols; ++j) {
            float acc = 0.0f;
            for (int64_t k = 0; k < rank; ++k) acc = fmaf(us[i * rank + k], vt[k * cols + j], acc);
            ker[i * cols + j] = acc;
        }
    return 0;
}

int metis_oracle_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
