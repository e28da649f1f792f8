/* Host checks of the arithmetic shortcuts the HIP quantizer kernels take (test infrastructure).
 *
 * The kernels do not run the reference's op sequence (src/Metis/Metis/quant.py:27-31) literally on
 * their fast paths; they use a 3-operation quotient, the hardware E2M1 converter (round to nearest
 * even onto the grid) and a few guards.  This program restates both sides in plain C and compares
 * them, exhaustively where the domain is small:
 *
 *   pb16        every op rounded to bf16: all (h, x) pairs of positive bf16 values with x/h in
 *               [0.05, 13.2]: literal sequence  vs  q = bf16(div3(x, h)), three q values nudged
 *               onto their tie, round-to-nearest-even onto the grid.
 *   div6        amax / 6 by a constant reciprocal and one correction: every finite non-negative bf16 value
 *               against the correctly rounded quotient (the block scalar, quant.py:19).
 *   p32 ITERS   binary32 arithmetic: for ITERS block scalars (realistic, random, and adversarially
 *               close to decision thresholds) and the bf16 inputs around every threshold:
 *               literal sequence  vs  round-to-nearest-even of div3(x, s), for blocks the kernel's
 *               two guards do not send to the literal path.
 *
 *   wide ITERS  binary32 arithmetic on binary32 values (not bf16 values): for ITERS block maxima of any
 *               significand, inputs anywhere below the maximum and the binary32 neighbours of every
 *               threshold: literal sequence  vs  round-to-nearest-even of div3(x, s), for quotients the
 *               kernel's per-element test does not send to the literal path.
 *
 *   table FILE  binary32 arithmetic on bf16 values with the two-operation quotient q = fma(x, rh, fma(x, rl, 0)): for every
 *               block maximum that the table in FILE (the kernels' quotient_table.h) clears, every bf16 element of such
 *               a block: literal sequence  vs  round-to-nearest-even of q.
 *
 * Exit status 0 and a final line "mismatches 0" mean the shortcut is exact on the domain covered.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static inline float bits_f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float rb(float f)                         /* round to nearest even bf16 */
{
    const uint32_t u = f_bits(f);
    return bits_f((u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u);
}
static inline float relu(float x) { return x > 0 ? x : 0; }

/* round to nearest even onto {0,1,2,3,4,6,8,12} (q units), returns the code 0..7 */
static int rne_grid(float q)
{
    static const double g[8] = {0, 1, 2, 3, 4, 6, 8, 12};
    const double y = fabs((double)q);
    int best = 0;
    double bd = 1e300;
    for (int i = 0; i < 8; i++) {
        const double d = fabs(y - g[i]);
        if (d < bd) { bd = d; best = i; }
        else if (d == bd && i % 2 == 0) best = i;
    }
    return best;
}
/* the kernels' 3-operation quotient (product, exact remainder, one correction) */
static inline float div3(float x, float s, float rs)
{
    const float w = x * rs;
    const float e = fmaf(-s, w, x);
    return fmaf(e, rs, w);
}

/* ---- every op rounded to bf16 (quant.py:27-31 on bf16 tensors) */
static int literal_pb16(float ax, float h)
{
    const float q = rb(ax / h);
    const float t1 = rb(rb(relu(rb(q - 4.0f))) / 2.0f);
    const float t2 = rb(rb(relu(rb(q - 8.0f))) / 4.0f);
    const float c = rb(q - rb(t1 + t2));
    float r = rintf(c);
    if (r > 7) r = 7;
    return (int)r;
}
static int shortcut_pb16(float ax, float h, int pert)
{
    const float rs = bits_f(f_bits(1.0f / h) + pert);     /* any reciprocal within 1 ulp */
    float q = rb(div3(ax, h, rs));
    if (q == 5.03125f) q = 5.0f;
    else if (q == 6.96875f) q = 7.0f;
    else if (q == 10.0625f) q = 10.0f;
    return rne_grid(q);
}
static long check_pb16(void)
{
    long n = 0, bad = 0;
#pragma omp parallel for reduction(+ : n, bad) schedule(dynamic, 64)
    for (uint32_t hp = 0x0080; hp < 0x7f80; ++hp) {
        const float h = bits_f(hp << 16), s = h * 2.0f;
        if (!(s < 3e38f)) continue;
        for (uint32_t xp = 0; xp < 0x7f80; ++xp) {
            const float x = bits_f(xp << 16);
            if (x > 6.6f * s) break;
            if (x < 0.05f * h) continue;
            const int want = literal_pb16(x, h);
            for (int pert = -1; pert <= 1; ++pert) {
                n++;
                if (shortcut_pb16(x, h, pert) != want) bad++;
            }
        }
    }
    printf("pb16: cases %ld mismatches %ld\n", n, bad);
    return bad;
}

/* ---- binary32 arithmetic */
static int literal_p32(float ax, float s)
{
    volatile float h = s / 2.0f;
    volatile float q = ax / h;
    volatile float a = relu(q - 4.0f) / 2.0f, b = relu(q - 8.0f) / 4.0f;
    volatile float c = a + b;
    volatile float qp = q - c;
    float r = rintf(qp);
    if (r > 7) r = 7;
    return (int)r;
}
/* the two guards of the kernels' binary32 fast path, restated */
static int may_hit_exception(float s)
{
    const float h = 0.5f * s;
    const float t5 = 5.0f * h, t7 = 7.0f * h;
    const uint32_t b5 = f_bits(t5), b7 = f_bits(t7);
    const int c5 = ((b5 + 4u) & 0xffffu) < 4u;
    const int c7 = ((b7 - 1u) & 0xffffu) < 4u;
    const int z5 = ((b5 & 0xffffu) == 0u) && (fmaf(5.0f, h, -t5) != 0.0f);
    const int z7 = ((b7 & 0xffffu) == 0u) && (fmaf(7.0f, h, -t7) != 0.0f);
    return c5 | c7 | z5 | z7;
}
static int near_threshold_hazard(float s)
{
    const uint32_t t = f_bits(s) & 0xfffffu;
    return (t != 0u) & (((t + 64u) & 0xfffffu) <= 128u);
}
static long check_p32(long iters)
{
    static const float W[7] = {0.25f, 0.75f, 1.25f, 1.75f, 2.5f, 3.5f, 5.0f};   /* thresholds in x/s units */
    long n = 0, bad = 0, guarded = 0;
#pragma omp parallel for reduction(+ : n, bad, guarded) schedule(dynamic, 1024)
    for (long it = 0; it < iters; ++it) {
        unsigned seed = 1234577u + 7919u * (unsigned)it + (unsigned)(it >> 20);
        const uint32_t r1 = rand_r(&seed), r2 = rand_r(&seed), r3 = rand_r(&seed);
        float s;
        switch (it % 4) {
        case 0: s = bits_f(((r1 % 0x4000) + 0x3000) << 16) / 6.0f + 1e-9f; break;                  /* amax/6 + 1e-9 */
        case 1: s = bits_f(((uint32_t)(100 + r2 % 60) << 23) | ((r1 ^ (r2 << 11)) & 0x7fffff)); break;
        case 2: s = bits_f(((uint32_t)(110 + r2 % 40) << 23) | ((r1 & 7) << 20) |
                           (r2 % 2 == 0 ? (r3 & 0xff) : (0xfffff - (r3 & 0xff)))); break;          /* low bits near 0 */
        default: {                                                                                /* W*s next to a bf16 value */
            const float xb = bits_f(((r2 % 0x3000) + 0x3800) << 16);
            s = bits_f(f_bits(xb / W[r1 % 7]) + (int)(r3 % 41) - 20);
        }
        }
        if (may_hit_exception(s) || near_threshold_hazard(s)) { guarded++; continue; }    /* kernel takes the literal path */
        const float rs0 = 1.0f / s;
        for (int wi = 0; wi < 7; ++wi) {
            const uint32_t cb = (f_bits(W[wi] * s) + 0x8000u) >> 16;
            for (int dx = -2; dx <= 2; ++dx) {
                const float x = bits_f((cb + dx) << 16);
                const int want = literal_p32(x, s);
                for (int pert = -1; pert <= 1; ++pert) {
                    const float q = div3(x, s, bits_f(f_bits(rs0) + pert));   /* x/s: half of the reference's q */
                    n++;
                    if (rne_grid(2.0f * q) != want) bad++;
                }
            }
        }
    }
    printf("p32: cases %ld (blocks sent to the literal path by the guards: %ld of %ld) mismatches %ld\n", n, guarded, iters, bad);
    return bad;
}

/* ---- binary32 arithmetic on binary32 VALUES (inputs that are not bf16 values): the block-level guards above do not
 * apply, the kernel tests every quotient instead: a quotient within 4 ulp of a value whose low 20 significand bits
 * are zero (every decision threshold is such a value) sends the block to the literal path. */
static int quotient_hazard(float q)
{
    uint32_t a = f_bits(q) & 0x7fffffffu;
    if (a < 0x3e000010u) a = 0x3e000010u;                         /* below 0.125 the code is 0 either way */
    if (a > 0x40b00010u) a = 0x40b00010u;                         /* above 5.5 it is 7 (every block maximum sits at 6) */
    return ((a + 4u) & 0xfffffu) < 8u;
}
static long check_wide(long iters)
{
    static const float W[7] = {0.25f, 0.75f, 1.25f, 1.75f, 2.5f, 3.5f, 5.0f};
    long n = 0, bad = 0, guarded = 0;
#pragma omp parallel for reduction(+ : n, bad, guarded) schedule(dynamic, 1024)
    for (long it = 0; it < iters; ++it) {
        unsigned seed = 99991u + 104729u * (unsigned)it + (unsigned)(it >> 18);
        const uint32_t r1 = rand_r(&seed), r2 = rand_r(&seed), r3 = rand_r(&seed), r4 = rand_r(&seed);
        /* a binary32 block maximum of any significand, and its scalar */
        const float amax = bits_f(((uint32_t)(90 + r2 % 70) << 23) | ((r1 ^ (r3 << 9)) & 0x7fffff));
        const float s = amax / 6.0f + 1e-9f;
        const float rs0 = 1.0f / s;
        for (int k = 0; k < 24; ++k) {
            float x;
            if (k < 8) {                                           /* anywhere below the maximum */
                const uint32_t rr = rand_r(&seed);
                x = amax * ((float)(rr & 0xffffff) / 16777216.0f);
            } else if (k < 22) {                                   /* binary32 neighbours of threshold * s */
                const float c = W[(k - 8) % 7] * s;
                x = bits_f(f_bits(c) + (int)(r4 >> (k - 8) & 15) - 8);
            } else {
                x = k == 22 ? amax : bits_f(f_bits(amax) - 1u);
            }
            if (!(x <= amax)) continue;
            const int want = literal_p32(x, s);
            for (int pert = -1; pert <= 1; ++pert) {
                const float q = div3(x, s, bits_f(f_bits(rs0) + pert));
                if (quotient_hazard(q)) { guarded++; continue; }
                n++;
                if (rne_grid(2.0f * q) != want) bad++;
            }
        }
    }
    printf("wide: cases %ld (quotients sent to the literal path: %ld) mismatches %ld\n", n, guarded, bad);
    return bad;
}

/* ---- binary32 arithmetic on bf16 values, two operations per quotient: the table of block maxima the kernels consult
 * (fp4-post_amd/csrc/quotient_table.h, one bit per bf16 pattern of the maximum).  For every maximum whose bit is set: every
 * bf16 element of such a block and the three reciprocals the hardware may return, against the literal sequence. */
static long check_table(const char* path)
{
    static uint32_t words[1024];
    FILE* f = fopen(path, "r");
    if (!f) { printf("table: cannot open %s\n", path); return 1; }
    char line[512];
    int nw = 0;
    while (fgets(line, sizeof line, f)) {
        if (strncmp(line, "0x", 2) != 0) continue;
        for (char* p = line; (p = strstr(p, "0x")) != NULL && nw < 1024; p += 2) words[nw++] = (uint32_t)strtoul(p, NULL, 16);
    }
    fclose(f);
    if (nw != 1024) { printf("table: %d words instead of 1024\n", nw); return 1; }
    long n = 0, bad = 0, set = 0;
#pragma omp parallel for reduction(+ : n, bad, set) schedule(dynamic, 64)
    for (uint32_t p = 0; p < 0x8000; ++p) {
        if (!((words[p >> 5] >> (p & 31)) & 1u)) continue;
        set++;
        if (p >= 0x7f80) { bad++; continue; }                   /* infinities and NaNs must never be cleared */
        const float amax = bits_f(p << 16);
        volatile float s0 = amax / 6.0f;
        volatile float s = s0 + 1e-9f;
        const float r0 = 1.0f / s;
        for (uint32_t xp = 0; xp <= p; ++xp) {
            const float x = bits_f(xp << 16);
            const int want = literal_p32(x, s);
            for (int pert = -1; pert <= 1; ++pert) {
                const float rh = bits_f(f_bits(r0) + pert);
                const float rl = fmaf(-s, rh, 1.0f) * rh;
                const float q = fmaf(x, rh, fmaf(x, rl, 0.0f));  /* x / s: half of the reference's quotient */
                n++;
                if (rne_grid(2.0f * q) != want) bad++;
            }
        }
    }
    printf("table: maxima cleared %ld, cases %ld mismatches %ld\n", set, n, bad);
    return bad;
}

static long check_div6(void)
{
    long n = 0, bad = 0;
    for (uint32_t p = 0; p < 0x7f80; ++p) {
        const float a = bits_f(p << 16), c = 0x1.555556p-3f;
        const float q = a * c;
        const float r = fmaf(-6.0f, q, a);
        n++;
        if (f_bits(fmaf(r, c, q)) != f_bits(a / 6.0f)) bad++;
    }
    printf("div6: cases %ld mismatches %ld\n", n, bad);
    return bad;
}

int main(int argc, char** argv)
{
    if (argc >= 2 && !strcmp(argv[1], "div6")) return check_div6() ? 1 : 0;
    if (argc >= 2 && !strcmp(argv[1], "pb16")) return check_pb16() ? 1 : 0;
    if (argc >= 3 && !strcmp(argv[1], "p32")) return check_p32(atol(argv[2])) ? 1 : 0;
    if (argc >= 3 && !strcmp(argv[1], "wide")) return check_wide(atol(argv[2])) ? 1 : 0;
    if (argc >= 3 && !strcmp(argv[1], "table")) return check_table(argv[2]) ? 1 : 0;
    fprintf(stderr, "usage: %s div6 | pb16 | p32 ITERS | wide ITERS | table QUOTIENT_TABLE_H\n", argv[0]);
    return 2;
}
