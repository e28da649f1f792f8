// Torch-free check of the C ABI: a plain C++ host program that owns its device memory through
// HIP, calls libmetis_hip.so the way a C caller of the library would, and compares with the C
// restatement of the reference arithmetic (oracle/libmetis_oracle.so, test infrastructure).
//
//   1. metis_nvfp4_quant_row in both parity modes  -> codes, scale bytes, unit bit-equal to the oracle
//   2. metis_rmsnorm_nvfp4_quant                   -> normed output and packed tensor bit-equal
//   3. metis_nvfp4_dequant                         -> bit-equal to the oracle's dequantization
//   4. metis_linear_fwd (tiled and skinny shapes)  -> against a double-precision product of the
//                                                     dequantized operands, rel. Frobenius error <= 2e-3
//   5. error codes for bad arguments
//   6. split-K through a caller workspace (metis_linear_fwd_ws: tiled and decode-sized shapes)
//   7. metis_linear_fwd_grouped, and metis_linear_fwd_grouped_centered with the centre from
//      metis_column_mean_running                    -> against double precision on the host
//   8. metis_nvfp4_matvec                           -> against double precision on the host
//
// Built and run by tests/test_gpu_cabi_native.py; prints one line per check and exits non-zero on failure.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <vector>

#include "metis_hip.h"

extern "C" {
uint16_t metis_oracle_f32_to_bf16(float f);
int metis_oracle_nvfp4_pack(const void* x, int64_t rows, int64_t cols, int64_t ld, int mode, const void* noise,
                            uint8_t* codes, uint8_t* scales, float* unit, int64_t* n_clamped);
int metis_oracle_nvfp4_dequant(const uint8_t* codes, const uint8_t* scales, float unit, int64_t rows, int64_t cols, int mode,
                               uint16_t* out_bf16, float* out_f32);
int metis_oracle_rmsnorm_nvfp4(const uint16_t* x, const uint16_t* gamma, float eps, int64_t rows, int64_t cols, int mode,
                               uint16_t* normed, uint8_t* codes, uint8_t* scales, float* unit);
}

#define HIP_OK(x)                                                                          \
    do {                                                                                   \
        hipError_t e_ = (x);                                                               \
        if (e_ != hipSuccess) {                                                            \
            printf("FAIL hip: %s at line %d\n", hipGetErrorString(e_), __LINE__);          \
            exit(2);                                                                       \
        }                                                                                  \
    } while (0)

static int failures = 0;
static void check(bool ok, const char* what)
{
    printf("%s %s\n", ok ? "ok  " : "FAIL", what);
    fflush(stdout);
    if (!ok) ++failures;
}

template <typename T>
struct DeviceBuffer {
    T* p = nullptr;
    size_t n = 0;
    explicit DeviceBuffer(size_t count) : n(count) { HIP_OK(hipMalloc(&p, count * sizeof(T) + 16)); }
    ~DeviceBuffer() { (void)hipFree(p); }
    void upload(const std::vector<T>& h) { HIP_OK(hipMemcpy(p, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice)); }
    std::vector<T> download() const
    {
        std::vector<T> h(n);
        HIP_OK(hipMemcpy(h.data(), p, n * sizeof(T), hipMemcpyDeviceToHost));
        return h;
    }
};

static float bf16_to_f32(uint16_t b)
{
    uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

// deterministic N(0,1)-ish bf16 data with an outlier column
static std::vector<uint16_t> make_input(int64_t rows, int64_t cols, unsigned seed, float scale)
{
    std::vector<uint16_t> x((size_t)(rows * cols));
    srand(seed);
    for (int64_t i = 0; i < rows * cols; ++i) {
        const double u1 = (rand() + 1.0) / (RAND_MAX + 2.0), u2 = rand() / (double)RAND_MAX;
        float v = (float)(sqrt(-2.0 * log(u1)) * cos(6.283185307179586 * u2)) * scale;
        if (i % cols == 5) v *= 20.0f;
        x[(size_t)i] = metis_oracle_f32_to_bf16(v);
    }
    return x;
}

struct Packed {
    std::vector<uint8_t> codes, scales;
    float unit;
};

static Packed quantize_on_device(const std::vector<uint16_t>& x, int64_t rows, int64_t cols, int mode, hipStream_t st,
                                 DeviceBuffer<uint8_t>* keep_codes = nullptr, DeviceBuffer<uint8_t>* keep_scales = nullptr,
                                 DeviceBuffer<float>* keep_unit = nullptr)
{
    DeviceBuffer<uint16_t> dx(x.size());
    dx.upload(x);
    DeviceBuffer<uint8_t> local_codes((size_t)(rows * cols / 2)), local_scales((size_t)(rows * cols / 16));
    DeviceBuffer<float> local_unit(1);
    DeviceBuffer<uint8_t>& dc = keep_codes ? *keep_codes : local_codes;
    DeviceBuffer<uint8_t>& ds = keep_scales ? *keep_scales : local_scales;
    DeviceBuffer<float>& du = keep_unit ? *keep_unit : local_unit;
    const size_t wsb = metis_nvfp4_workspace_bytes(rows, cols);
    DeviceBuffer<uint8_t> ws(wsb);
    HIP_OK(hipMemset(ws.p, 0, wsb));                            // zero-filled once, as the contract asks
    const int rc = metis_nvfp4_quant_row(dx.p, rows, cols, cols, mode, dc.p, ds.p, du.p, ws.p, wsb, st);
    if (rc != METIS_OK) {
        printf("FAIL metis_nvfp4_quant_row rc=%d (%s)\n", rc, metis_error_string(rc));
        exit(2);
    }
    HIP_OK(hipStreamSynchronize(st));
    Packed p;
    p.codes = dc.download();
    p.scales = ds.download();
    p.unit = du.download()[0];
    return p;
}

static double rel_fro(const std::vector<double>& got, const std::vector<double>& want)
{
    double num = 0, den = 0;
    for (size_t i = 0; i < got.size(); ++i) {
        num += (got[i] - want[i]) * (got[i] - want[i]);
        den += want[i] * want[i];
    }
    return sqrt(num / (den > 0 ? den : 1));
}

static void check_linear(int64_t M, int64_t N, int64_t K, hipStream_t st, const char* what, bool with_workspace = false)
{
    const std::vector<uint16_t> x = make_input(M, K, 11u + (unsigned)M, 1.0f), w = make_input(N, K, 12u + (unsigned)N, 0.02f);
    DeviceBuffer<uint8_t> ac((size_t)(M * K / 2)), as((size_t)(M * K / 16)), bc((size_t)(N * K / 2)), bs((size_t)(N * K / 16));
    DeviceBuffer<float> au(1), bu(1);
    const Packed pa = quantize_on_device(x, M, K, METIS_MODE_P32, st, &ac, &as, &au);
    const Packed pb = quantize_on_device(w, N, K, METIS_MODE_P32, st, &bc, &bs, &bu);
    DeviceBuffer<float> out((size_t)(M * N));
    int rc;
    if (with_workspace) {
        const size_t need = metis_linear_workspace_bytes(M, N, K);
        char l2[160];
        snprintf(l2, sizeof l2, "%s: metis_linear_workspace_bytes = %zu (the shape is split)", what, need);
        check(need > 0, l2);
        DeviceBuffer<uint8_t> ws(need ? need : 16);              // no initialisation needed
        rc = metis_linear_fwd_ws(ac.p, as.p, au.p, bc.p, bs.p, bu.p, M, N, K, nullptr, nullptr, 0, nullptr, out.p, METIS_DTYPE_F32,
                                 ws.p, need, st);
        HIP_OK(hipStreamSynchronize(st));
    } else {
        rc = metis_linear_fwd(ac.p, as.p, au.p, bc.p, bs.p, bu.p, M, N, K, nullptr, nullptr, 0, nullptr, out.p, METIS_DTYPE_F32, st);
        HIP_OK(hipStreamSynchronize(st));
    }
    std::vector<float> xa((size_t)(M * K)), wb((size_t)(N * K));
    metis_oracle_nvfp4_dequant(pa.codes.data(), pa.scales.data(), pa.unit, M, K, 0, nullptr, xa.data());
    metis_oracle_nvfp4_dequant(pb.codes.data(), pb.scales.data(), pb.unit, N, K, 0, nullptr, wb.data());
    std::vector<double> want((size_t)(M * N)), got((size_t)(M * N));
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            double s = 0;
            for (int64_t k = 0; k < K; ++k) s += (double)xa[(size_t)(m * K + k)] * (double)wb[(size_t)(n * K + k)];
            want[(size_t)(m * N + n)] = s;
        }
    const std::vector<float> o = out.download();
    for (size_t i = 0; i < o.size(); ++i) got[i] = o[i];
    const double err = rel_fro(got, want);
    char line[160];
    snprintf(line, sizeof line, "%s: metis_linear_fwd %ldx%ldx%ld rc=%d rel.err %.2e", what, (long)M, (long)N, (long)K, rc, err);
    check(rc == METIS_OK && err <= 2e-3, line);
}

// The pipelined GEMM on tiled 16-bit expansions: metis_nvfp4_expand_tiled for both operands, metis_linear_fwd_tiled,
// against the packed-operand GEMM on the same packed tensors (same products, binary32 sums in another order) and, with
// the rotated quantizer, the NV recipe's round trip: quant_row_rht -> dequant -> hadamard16 (inverse) stays close to x.
static void check_tiled(int64_t M, int64_t N, int64_t K, hipStream_t st)
{
    const std::vector<uint16_t> x = make_input(M, K, 21u, 1.0f), w = make_input(N, K, 22u, 0.02f);
    DeviceBuffer<uint8_t> ac((size_t)(M * K / 2)), as((size_t)(M * K / 16)), bc((size_t)(N * K / 2)), bs((size_t)(N * K / 16));
    DeviceBuffer<float> au(1), bu(1);
    quantize_on_device(x, M, K, METIS_MODE_P32, st, &ac, &as, &au);
    quantize_on_device(w, N, K, METIS_MODE_P32, st, &bc, &bs, &bu);
    DeviceBuffer<uint8_t> ax(metis_nvfp4_expand_tiled_bytes(M, K)), bx(metis_nvfp4_expand_tiled_bytes(N, K));
    int rc = metis_nvfp4_expand_tiled(ac.p, as.p, au.p, M, K, METIS_MODE_P32, ax.p, st);
    if (rc == METIS_OK) rc = metis_nvfp4_expand_tiled(bc.p, bs.p, bu.p, N, K, METIS_MODE_P32, bx.p, st);
    DeviceBuffer<float> out_t((size_t)(M * N)), out_p((size_t)(M * N));
    const size_t need = metis_linear_tiled_workspace_bytes(M, N, K, METIS_MODE_P32);
    DeviceBuffer<uint8_t> ws(need ? need : 16);
    if (rc == METIS_OK)
        rc = metis_linear_fwd_tiled(ax.p, au.p, bx.p, bu.p, M, N, K, nullptr, nullptr, 0, nullptr, 0, out_t.p, METIS_DTYPE_F32, METIS_MODE_P32,
                                    need ? ws.p : nullptr, need, st);
    if (rc == METIS_OK) rc = metis_linear_fwd(ac.p, as.p, au.p, bc.p, bs.p, bu.p, M, N, K, nullptr, nullptr, 0, nullptr, out_p.p, METIS_DTYPE_F32, st);
    HIP_OK(hipStreamSynchronize(st));
    const std::vector<float> t = out_t.download(), q = out_p.download();
    std::vector<double> got(t.begin(), t.end()), want(q.begin(), q.end());
    char line[200];
    snprintf(line, sizeof line, "metis_nvfp4_expand_tiled + metis_linear_fwd_tiled %ldx%ldx%ld rc=%d vs metis_linear_fwd rel.err %.2e",
             (long)M, (long)N, (long)K, rc, rel_fro(got, want));
    check(rc == METIS_OK && rel_fro(got, want) <= 1e-6, line);

    // NV recipe round trip on the activation (sign mask 0x5a3c: any mask is a valid rotation)
    DeviceBuffer<uint16_t> dx(x.size()), deq(x.size()), back(x.size());
    dx.upload(x);
    const size_t wsb = metis_nvfp4_workspace_bytes(M, K);
    DeviceBuffer<uint8_t> qws(wsb);
    HIP_OK(hipMemset(qws.p, 0, wsb));
    rc = metis_nvfp4_quant_row_rht(dx.p, M, K, K, METIS_MODE_PB16, 0x5a3cu, 0, 0, 0, ac.p, as.p, au.p, qws.p, wsb, st);
    if (rc == METIS_OK) rc = metis_nvfp4_dequant(ac.p, as.p, au.p, M, K, METIS_MODE_PB16, deq.p, METIS_DTYPE_BF16, st);
    if (rc == METIS_OK) rc = metis_hadamard16(deq.p, M, K, K, METIS_DTYPE_BF16, 1, 0x5a3cu, back.p, K, st);
    HIP_OK(hipStreamSynchronize(st));
    const std::vector<uint16_t> b = back.download();
    std::vector<double> g2(b.size()), w2(b.size());
    for (size_t i = 0; i < b.size(); ++i) { g2[i] = bf16_to_f32(b[i]); w2[i] = bf16_to_f32(x[i]); }
    snprintf(line, sizeof line, "metis_nvfp4_quant_row_rht -> dequant -> metis_hadamard16 (inverse) rc=%d rel.err to x %.3f (FP4 level)", rc,
             rel_fro(g2, w2));
    check(rc == METIS_OK && rel_fro(g2, w2) < 0.2, line);
    check(metis_nvfp4_quant_row_rht(dx.p, M, K, K, METIS_MODE_PB16, 0x10000u, 0, 0, 0, ac.p, as.p, au.p, qws.p, wsb, st) == METIS_E_ARG,
          "a sign mask wider than 16 bits -> METIS_E_ARG");
}

// bf16 arithmetic at decode size: metis_linear_fwd_grouped_bf16 on the packed activation and
// metis_nvfp4_decode_operand + metis_linear_fwd_grouped_operand give the same bits, and both agree with the all-bf16
// evaluation (bf16 dequantized operands from metis_nvfp4_dequant, product rounded to bf16) computed on the host.
static void check_decode_bf16(int64_t M, int64_t N, int64_t K, hipStream_t st)
{
    const std::vector<uint16_t> x = make_input(M, K, 31u, 1.0f), w = make_input(N, K, 32u, 0.02f);
    DeviceBuffer<uint8_t> ac((size_t)(M * K / 2)), as((size_t)(M * K / 16)), bc((size_t)(N * K / 2)), bs((size_t)(N * K / 16));
    DeviceBuffer<float> au(1), bu(1);
    quantize_on_device(x, M, K, METIS_MODE_PB16, st, &ac, &as, &au);
    quantize_on_device(w, N, K, METIS_MODE_PB16, st, &bc, &bs, &bu);
    DeviceBuffer<uint16_t> xa((size_t)(M * K)), wb((size_t)(N * K)), out_a((size_t)(M * N)), out_b((size_t)(M * N));
    int rc = metis_nvfp4_dequant(ac.p, as.p, au.p, M, K, METIS_MODE_PB16, xa.p, METIS_DTYPE_BF16, st);
    if (rc == METIS_OK) rc = metis_nvfp4_dequant(bc.p, bs.p, bu.p, N, K, METIS_MODE_PB16, wb.p, METIS_DTYPE_BF16, st);
    metis_linear_member mem = {};
    mem.b_codes = bc.p; mem.b_scales = bs.p; mem.b_unit = bu.p; mem.N = N;
    const size_t need = metis_linear_grouped_workspace_bytes(M, K, &mem, 1);
    DeviceBuffer<uint8_t> ws(need ? need : 16), aop(metis_nvfp4_decode_operand_bytes(M, K));
    mem.out = out_a.p;
    if (rc == METIS_OK) rc = metis_linear_fwd_grouped_bf16(ac.p, as.p, au.p, M, K, &mem, 1, METIS_DTYPE_BF16, need ? ws.p : nullptr, need, st);
    mem.out = out_b.p;
    if (rc == METIS_OK) rc = metis_nvfp4_decode_operand(ac.p, as.p, au.p, M, K, METIS_MODE_PB16, nullptr, aop.p, st);
    if (rc == METIS_OK)
        rc = metis_linear_fwd_grouped_operand(aop.p, au.p, M, K, &mem, 1, METIS_DTYPE_BF16, METIS_MODE_PB16, need ? ws.p : nullptr, need, st);
    HIP_OK(hipStreamSynchronize(st));
    const std::vector<uint16_t> a = out_a.download(), b = out_b.download(), xq = xa.download(), wq = wb.download();
    size_t differ = 0, off = 0;
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            double s = 0;
            for (int64_t k = 0; k < K; ++k) s += (double)bf16_to_f32(xq[(size_t)(m * K + k)]) * (double)bf16_to_f32(wq[(size_t)(n * K + k)]);
            const float f = (float)s;
            uint32_t u;
            memcpy(&u, &f, 4);
            const uint16_t want = (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);      // round to nearest even
            differ += a[(size_t)(m * N + n)] != b[(size_t)(m * N + n)];
            off += a[(size_t)(m * N + n)] != want;
        }
    char line[240];
    snprintf(line, sizeof line, "metis_linear_fwd_grouped_bf16 vs decode operand path %ldx%ldx%ld rc=%d: %zu differ; %zu of %ld off the all-bf16 "
             "evaluation (sums on a rounding boundary)", (long)M, (long)N, (long)K, rc, differ, off, (long)(M * N));
    check(rc == METIS_OK && differ == 0 && off * 500 <= (size_t)(M * N), line);
    check(metis_linear_fwd_grouped_bf16(ac.p, as.p, au.p, 256, K, &mem, 1, METIS_DTYPE_BF16, nullptr, 0, st) == METIS_E_ARG,
          "metis_linear_fwd_grouped_bf16 with 256 rows -> METIS_E_ARG (the pipelined kernel's size)");
}

// NV recipe at decode size: a weight packed in the rotated domain is streamed as it is by the decode-sized kernel and
// the activation's operand carries the rotation (metis_nvfp4_decode_operand_rht).  Against the double-precision product
// of the activation's dequantized values (oracle) with the weight dequantized and rotated back
// (metis_nvfp4_dequant + metis_hadamard16, binary32), in binary32 arithmetic: one binary16 rounding of the rotated operand.
static void check_decode_rotated_weight(int64_t M, int64_t N, int64_t K, hipStream_t st)
{
    const uint32_t mask = 0x5a3cu;
    const std::vector<uint16_t> x = make_input(M, K, 51u, 1.0f), w = make_input(N, K, 52u, 0.02f);
    DeviceBuffer<uint16_t> dw(w.size());
    dw.upload(w);
    DeviceBuffer<uint8_t> ac((size_t)(M * K / 2)), as((size_t)(M * K / 16)), bc((size_t)(N * K / 2)), bs((size_t)(N * K / 16));
    DeviceBuffer<float> au(1), bu(1), wdeq((size_t)(N * K)), wback((size_t)(N * K)), out((size_t)(M * N));
    const Packed pa = quantize_on_device(x, M, K, METIS_MODE_P32, st, &ac, &as, &au);
    const size_t wsb = metis_nvfp4_workspace_bytes(N, K);
    DeviceBuffer<uint8_t> qws(wsb), aop(metis_nvfp4_decode_operand_bytes(M, K));
    HIP_OK(hipMemset(qws.p, 0, wsb));
    int rc = metis_nvfp4_quant_row_rht(dw.p, N, K, K, METIS_MODE_P32, mask, 0, 0, 0, bc.p, bs.p, bu.p, qws.p, wsb, st);
    if (rc == METIS_OK) rc = metis_nvfp4_dequant(bc.p, bs.p, bu.p, N, K, METIS_MODE_P32, wdeq.p, METIS_DTYPE_F32, st);
    if (rc == METIS_OK) rc = metis_hadamard16(wdeq.p, N, K, K, METIS_DTYPE_F32, 1, mask, wback.p, K, st);
    if (rc == METIS_OK) rc = metis_nvfp4_decode_operand_rht(ac.p, as.p, au.p, nullptr, M, K, METIS_MODE_P32, METIS_MODE_P32, mask, aop.p, st);
    metis_linear_member mem = {};
    mem.b_codes = bc.p; mem.b_scales = bs.p; mem.b_unit = bu.p; mem.N = N; mem.out = out.p;
    const size_t need = metis_linear_grouped_workspace_bytes(M, K, &mem, 1);
    DeviceBuffer<uint8_t> gws(need ? need : 16);
    if (rc == METIS_OK)
        rc = metis_linear_fwd_grouped_operand(aop.p, au.p, M, K, &mem, 1, METIS_DTYPE_F32, METIS_MODE_P32, need ? gws.p : nullptr, need, st);
    HIP_OK(hipStreamSynchronize(st));
    std::vector<float> xa((size_t)(M * K));
    metis_oracle_nvfp4_dequant(pa.codes.data(), pa.scales.data(), pa.unit, M, K, 0, nullptr, xa.data());
    const std::vector<float> wb = wback.download(), got_f = out.download();
    std::vector<double> got(got_f.begin(), got_f.end()), want((size_t)(M * N));
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            double sum = 0;
            for (int64_t k = 0; k < K; ++k) sum += (double)xa[(size_t)(m * K + k)] * (double)wb[(size_t)(n * K + k)];
            want[(size_t)(m * N + n)] = sum;
        }
    char line[240];
    snprintf(line, sizeof line, "metis_nvfp4_decode_operand_rht + grouped operand call %ldx%ldx%ld rc=%d vs x^ . rotate_back(Q)^T rel.err %.2e",
             (long)M, (long)N, (long)K, rc, rel_fro(got, want));
    check(rc == METIS_OK && rel_fro(got, want) <= 5e-4, line);
    check(metis_nvfp4_decode_operand_rht(ac.p, as.p, au.p, nullptr, M, K, METIS_MODE_P32, METIS_MODE_P32, 0x10000u, aop.p, st) == METIS_E_ARG,
          "metis_nvfp4_decode_operand_rht with a sign mask wider than 16 bits -> METIS_E_ARG");
    check(metis_nvfp4_decode_operand_rht(ac.p, as.p, au.p, nullptr, 256, K, METIS_MODE_P32, METIS_MODE_P32, mask, aop.p, st) == METIS_E_SHAPE,
          "metis_nvfp4_decode_operand_rht with 256 rows -> METIS_E_SHAPE");
}

// A decode-sized BitLinear.forward in bf16 arithmetic as three launches: quantizer + the projection's first step,
// its finishing step + the activation's GEMM operands, the GEMM.  The quantizer's half against the C oracle, the
// projection against double precision on the host, the output against the same forward through the separate calls.
static void check_decode_three_launches(int64_t M, int64_t N, int64_t K, int64_t R, hipStream_t st)
{
    const std::vector<uint16_t> x = make_input(M, K, 41u, 1.0f), w = make_input(N, K, 42u, 0.02f), v = make_input(R, K, 43u, 0.02f);
    std::vector<uint16_t> sv((size_t)R), u = make_input(N, R, 44u, 0.1f);
    for (int64_t j = 0; j < R; ++j) sv[(size_t)j] = metis_oracle_f32_to_bf16(0.5f + 0.01f * (float)j);
    DeviceBuffer<uint16_t> dx(x.size()), dv(v.size()), ds(sv.size()), du(u.size());
    dx.upload(x); dv.upload(v); ds.upload(sv); du.upload(u);
    DeviceBuffer<uint8_t> bc((size_t)(N * K / 2)), bs((size_t)(N * K / 16));
    DeviceBuffer<float> bu(1);
    quantize_on_device(w, N, K, METIS_MODE_PB16, st, &bc, &bs, &bu);
    // merged launches
    DeviceBuffer<uint8_t> codes((size_t)(M * K / 2)), parked(metis_nvfp4_deferred_bytes(M, K) + 256);
    uint8_t* parked_p = (uint8_t*)(((uintptr_t)parked.p + 255) & ~(uintptr_t)255);
    const size_t lws = metis_lowrank_project_workspace_bytes(M, R, K);
    DeviceBuffer<uint8_t> lr_ws(lws), aop(metis_nvfp4_decode_operand_bytes(M, K));
    DeviceBuffer<uint16_t> xv((size_t)(M * R)), t((size_t)(M * R)), out_a((size_t)(M * N)), out_b((size_t)(M * N));
    DeviceBuffer<float> unit(1);
    int rc = metis_decode_quant_project_deferred(dx.p, M, K, METIS_MODE_PB16, codes.p, parked_p, metis_nvfp4_deferred_bytes(M, K), dv.p, R,
                                                 lr_ws.p, lws, st);
    if (rc == METIS_OK)
        rc = metis_decode_prepare_deferred(nullptr, K, dv.p, R, ds.p, xv.p, t.p, lr_ws.p, lws, codes.p, parked_p, M, K, METIS_MODE_PB16,
                                           METIS_MODE_PB16, nullptr, unit.p, aop.p, 0, 0u, st);
    metis_linear_member mem = {};
    mem.b_codes = bc.p; mem.b_scales = bs.p; mem.b_unit = bu.p; mem.N = N; mem.t = t.p; mem.u = du.p; mem.r = (int)R;
    const size_t need = metis_linear_grouped_workspace_bytes(M, K, &mem, 1);
    DeviceBuffer<uint8_t> gws(need ? need : 16);
    mem.out = out_a.p;
    if (rc == METIS_OK)
        rc = metis_linear_fwd_grouped_operand(aop.p, unit.p, M, K, &mem, 1, METIS_DTYPE_BF16, METIS_MODE_PB16, need ? gws.p : nullptr, need, st);
    HIP_OK(hipStreamSynchronize(st));
    // the quantizer's half against the oracle (codes and tensor unit; the scale bytes are never written on this path)
    std::vector<uint8_t> wc((size_t)(M * K / 2)), wsc((size_t)(M * K / 16));
    float wu = 0.0f;
    metis_oracle_nvfp4_pack(x.data(), M, K, K, METIS_MODE_PB16, nullptr, wc.data(), wsc.data(), &wu, nullptr);
    char line[260];
    snprintf(line, sizeof line, "metis_decode_quant_project_deferred %ldx%ld r=%ld rc=%d: codes and unit equal the oracle's", (long)M, (long)K, (long)R, rc);
    check(rc == METIS_OK && codes.download() == wc && unit.download()[0] == wu, line);
    // the projection against double precision: one bf16 rounding of the exact sum, t = bf16(xv * s)
    const std::vector<uint16_t> gxv = xv.download(), gt = t.download();
    double worst = 0.0, scale = 0.0;
    size_t t_off = 0;
    for (int64_t m = 0; m < M; ++m)
        for (int64_t j = 0; j < R; ++j) {
            double sum = 0;
            for (int64_t k = 0; k < K; ++k) sum += (double)bf16_to_f32(x[(size_t)(m * K + k)]) * (double)bf16_to_f32(v[(size_t)(j * K + k)]);
            worst = fmax(worst, fabs((double)bf16_to_f32(gxv[(size_t)(m * R + j)]) - sum));
            scale = fmax(scale, fabs(sum));
            t_off += gt[(size_t)(m * R + j)] != metis_oracle_f32_to_bf16(bf16_to_f32(gxv[(size_t)(m * R + j)]) * bf16_to_f32(sv[(size_t)j]));
        }
    snprintf(line, sizeof line, "metis_decode_prepare_deferred: x V^T within a bf16 ulp of the exact sums (%.3g of max %.3g), t = bf16(xv * s) (%zu off)",
             worst, scale, t_off);
    check(worst <= scale / 128.0 && t_off == 0, line);
    // the same forward through the separate calls
    DeviceBuffer<uint8_t> ac((size_t)(M * K / 2)), as((size_t)(M * K / 16)), aop2(metis_nvfp4_decode_operand_bytes(M, K)), lr_ws2(lws);
    DeviceBuffer<float> au(1);
    DeviceBuffer<uint16_t> xv2((size_t)(M * R)), t2((size_t)(M * R));
    quantize_on_device(x, M, K, METIS_MODE_PB16, st, &ac, &as, &au);
    int rc2 = metis_lowrank_project(dx.p, K, dv.p, M, R, K, ds.p, xv2.p, t2.p, lr_ws2.p, lws, st);
    if (rc2 == METIS_OK) rc2 = metis_nvfp4_decode_operand(ac.p, as.p, au.p, M, K, METIS_MODE_PB16, nullptr, aop2.p, st);
    mem.t = t2.p; mem.out = out_b.p;
    if (rc2 == METIS_OK)
        rc2 = metis_linear_fwd_grouped_operand(aop2.p, au.p, M, K, &mem, 1, METIS_DTYPE_BF16, METIS_MODE_PB16, need ? gws.p : nullptr, need, st);
    HIP_OK(hipStreamSynchronize(st));
    snprintf(line, sizeof line, "decode-sized forward %ldx%ldx%ld r=%ld in three launches equals the separate calls bit for bit (rc %d, %d)",
             (long)M, (long)N, (long)K, (long)R, rc, rc2);
    check(rc == METIS_OK && rc2 == METIS_OK && out_a.download() == out_b.download() && xv2.download() == gxv && aop2.download() == aop.download(), line);
    check(metis_decode_quant_project_deferred(dx.p, 256, K, METIS_MODE_PB16, codes.p, parked_p, metis_nvfp4_deferred_bytes(M, K), dv.p, R, lr_ws.p,
                                              lws, st) == METIS_E_SHAPE, "metis_decode_quant_project_deferred with 256 rows -> METIS_E_SHAPE");
}

// Mean mode at decode size: column mean (with the running update) -> centred quantizer -> grouped GEMM with the
// centre inside, and the packed matrix-vector product, all against double precision on the host.
static void check_mean_mode_decode(hipStream_t st)
{
    const int64_t M = 24, K = 512, N0 = 96, N1 = 36;
    std::vector<uint16_t> x = make_input(M, K, 21u, 1.0f);
    for (size_t i = 0; i < x.size(); ++i) x[i] = metis_oracle_f32_to_bf16(bf16_to_f32(x[i]) + 0.75f);      // an offset worth removing
    const std::vector<uint16_t> w0 = make_input(N0, K, 22u, 0.05f), w1 = make_input(N1, K, 23u, 0.05f);
    DeviceBuffer<uint16_t> dx(x.size());
    dx.upload(x);
    // running mean in binary32: cached = 0.5 for every column with weight 40 rows
    std::vector<float> cached((size_t)K, 0.5f);
    DeviceBuffer<float> dcached((size_t)K), dme((size_t)K);
    dcached.upload(cached);
    const size_t mws = metis_column_mean_workspace_bytes(K);
    DeviceBuffer<uint8_t> ws_mean(mws);
    int rc = metis_column_mean_running(dx.p, M, K, K, METIS_DTYPE_BF16, dcached.p, 40, dme.p, nullptr, METIS_DTYPE_F32, ws_mean.p, mws, st);
    HIP_OK(hipStreamSynchronize(st));
    const std::vector<float> me = dme.download();
    double worst = 0;
    for (int64_t c = 0; c < K; ++c) {
        double sum = 0;
        for (int64_t r = 0; r < M; ++r) sum += bf16_to_f32(x[(size_t)(r * K + c)]);
        const double want = (0.5 * 40 + (sum / M) * M) / (40 + M);
        worst = fmax(worst, fabs(me[(size_t)c] - want));
    }
    char line[200];
    snprintf(line, sizeof line, "metis_column_mean_running rc=%d: weighted running mean, worst abs. error %.2e", rc, worst);
    check(rc == METIS_OK && worst <= 1e-6, line);

    // centred quantizer: the packed tensor is that of x - me (binary32 arithmetic)
    DeviceBuffer<uint8_t> ac((size_t)(M * K / 2)), as((size_t)(M * K / 16));
    DeviceBuffer<float> au(1);
    const size_t qws = metis_nvfp4_workspace_bytes(M, K);
    DeviceBuffer<uint8_t> ws_q(qws);
    HIP_OK(hipMemset(ws_q.p, 0, qws));
    rc = metis_nvfp4_quant_centered(dx.p, M, K, K, METIS_MODE_P32, dme.p, 0, 0, nullptr, 0, 0, ac.p, as.p, au.p, ws_q.p, qws, st);
    HIP_OK(hipStreamSynchronize(st));
    std::vector<float> res((size_t)(M * K));
    for (int64_t r = 0; r < M; ++r)
        for (int64_t c = 0; c < K; ++c) res[(size_t)(r * K + c)] = bf16_to_f32(x[(size_t)(r * K + c)]) - me[(size_t)c];
    std::vector<uint8_t> wc((size_t)(M * K / 2)), wsc((size_t)(M * K / 16));
    float wu = 0;
    metis_oracle_nvfp4_pack(res.data(), M, K, K, 2, nullptr, wc.data(), wsc.data(), &wu, nullptr);      // mode 2: binary32 input
    check(rc == METIS_OK && ac.download() == wc && as.download() == wsc && au.download()[0] == wu,
          "metis_nvfp4_quant_centered: packed residual bit-equal to the oracle on x - me");
    std::vector<float> rdq((size_t)(M * K));
    metis_oracle_nvfp4_dequant(wc.data(), wsc.data(), wu, M, K, 0, nullptr, rdq.data());

    // two weights, one launch, the centre inside
    DeviceBuffer<uint8_t> b0c((size_t)(N0 * K / 2)), b0s((size_t)(N0 * K / 16)), b1c((size_t)(N1 * K / 2)), b1s((size_t)(N1 * K / 16));
    DeviceBuffer<float> b0u(1), b1u(1), o0((size_t)(M * N0)), o1((size_t)(M * N1));
    const Packed p0 = quantize_on_device(w0, N0, K, METIS_MODE_P32, st, &b0c, &b0s, &b0u);
    const Packed p1 = quantize_on_device(w1, N1, K, METIS_MODE_P32, st, &b1c, &b1s, &b1u);
    metis_linear_member mem[2] = {};
    mem[0].b_codes = b0c.p; mem[0].b_scales = b0s.p; mem[0].b_unit = b0u.p; mem[0].out = o0.p; mem[0].N = N0;
    mem[1].b_codes = b1c.p; mem[1].b_scales = b1s.p; mem[1].b_unit = b1u.p; mem[1].out = o1.p; mem[1].N = N1;
    const size_t gneed = metis_linear_grouped_workspace_bytes(M, K, mem, 2);
    DeviceBuffer<uint8_t> gws(gneed ? gneed : 16);
    const int supported = metis_linear_grouped_centered_supported(M, K, mem, 2, gneed > 0);
    check(supported == 1, "metis_linear_grouped_centered_supported for a decode-sized group");
    rc = metis_linear_fwd_grouped_centered(ac.p, as.p, au.p, M, K, mem, 2, METIS_DTYPE_F32, dme.p, gneed ? gws.p : nullptr, gneed, st);
    HIP_OK(hipStreamSynchronize(st));
    const Packed* pw[2] = {&p0, &p1};
    const int64_t Ns[2] = {N0, N1};
    const std::vector<float> got_o[2] = {o0.download(), o1.download()};
    for (int g = 0; g < 2; ++g) {
        std::vector<float> wdq((size_t)(Ns[g] * K));
        metis_oracle_nvfp4_dequant(pw[g]->codes.data(), pw[g]->scales.data(), pw[g]->unit, Ns[g], K, 0, nullptr, wdq.data());
        std::vector<double> want((size_t)(M * Ns[g])), got((size_t)(M * Ns[g]));
        for (int64_t m = 0; m < M; ++m)
            for (int64_t n = 0; n < Ns[g]; ++n) {
                double sacc = 0;
                for (int64_t k = 0; k < K; ++k) sacc += ((double)rdq[(size_t)(m * K + k)] + me[(size_t)k]) * wdq[(size_t)(n * K + k)];
                want[(size_t)(m * Ns[g] + n)] = sacc;
                got[(size_t)(m * Ns[g] + n)] = got_o[g][(size_t)(m * Ns[g] + n)];
            }
        const double err = rel_fro(got, want);
        snprintf(line, sizeof line, "metis_linear_fwd_grouped_centered member %d (%ldx%ldx%ld) rc=%d rel.err %.2e", g, (long)M, (long)Ns[g], (long)K, rc, err);
        check(rc == METIS_OK && err <= 5e-5, line);
    }
    // the same group without the centre equals R W^T
    rc = metis_linear_fwd_grouped(ac.p, as.p, au.p, M, K, mem, 2, METIS_DTYPE_F32, nullptr, 0, st);
    HIP_OK(hipStreamSynchronize(st));
    {
        std::vector<float> wdq((size_t)(N1 * K));
        metis_oracle_nvfp4_dequant(p1.codes.data(), p1.scales.data(), p1.unit, N1, K, 0, nullptr, wdq.data());
        const std::vector<float> o = o1.download();
        std::vector<double> want((size_t)(M * N1)), got((size_t)(M * N1));
        for (int64_t m = 0; m < M; ++m)
            for (int64_t n = 0; n < N1; ++n) {
                double sacc = 0;
                for (int64_t k = 0; k < K; ++k) sacc += (double)rdq[(size_t)(m * K + k)] * wdq[(size_t)(n * K + k)];
                want[(size_t)(m * N1 + n)] = sacc;
                got[(size_t)(m * N1 + n)] = o[(size_t)(m * N1 + n)];
            }
        const double err = rel_fro(got, want);
        snprintf(line, sizeof line, "metis_linear_fwd_grouped member 1 rc=%d rel.err %.2e", rc, err);
        check(rc == METIS_OK && err <= 5e-5, line);
    }
    // packed matrix-vector product: W^_0 me
    DeviceBuffer<float> dy((size_t)N0);
    rc = metis_nvfp4_matvec(b0c.p, b0s.p, b0u.p, N0, K, dme.p, 1.0f, dy.p, nullptr, 0, 0, st);
    HIP_OK(hipStreamSynchronize(st));
    {
        std::vector<float> wdq((size_t)(N0 * K));
        metis_oracle_nvfp4_dequant(p0.codes.data(), p0.scales.data(), p0.unit, N0, K, 0, nullptr, wdq.data());
        const std::vector<float> y = dy.download();
        std::vector<double> want((size_t)N0), got((size_t)N0);
        for (int64_t n = 0; n < N0; ++n) {
            double sacc = 0;
            for (int64_t k = 0; k < K; ++k) sacc += (double)wdq[(size_t)(n * K + k)] * me[(size_t)k];
            want[(size_t)n] = sacc;
            got[(size_t)n] = y[(size_t)n];
        }
        const double err = rel_fro(got, want);
        snprintf(line, sizeof line, "metis_nvfp4_matvec rc=%d rel.err %.2e", rc, err);
        check(rc == METIS_OK && err <= 1e-5, line);
    }
}

// One pass over an activation: NVFP4 codes + parked maxima (scale bytes formed afterwards) and the rank-r projection.
static void check_quant_project(int64_t M, int64_t K, int64_t R, int mode, hipStream_t st)
{
    const std::vector<uint16_t> x = make_input(M, K, 7u + (unsigned)M, 1.0f), v = make_input(R, K, 8u, 0.05f), s = make_input(1, R, 9u, 1.0f);
    DeviceBuffer<uint16_t> dx(x.size()), dv(v.size()), dsv(s.size()), dxv((size_t)(M * R)), dt((size_t)(M * R));
    dx.upload(x); dv.upload(v); dsv.upload(s);
    DeviceBuffer<uint8_t> dc((size_t)(M * K / 2)), dsc((size_t)(M * K / 16));
    DeviceBuffer<float> du(1);
    const size_t pb = metis_nvfp4_deferred_bytes(M, K), wb = metis_lowrank_project_rows_workspace_bytes(M, R, K);
    DeviceBuffer<uint8_t> parked(pb), ws(wb + 16);
    int rc = metis_nvfp4_quant_project_deferred(dx.p, M, K, mode, dv.p, R, dsv.p, dxv.p, dt.p, dc.p, parked.p, pb, wb ? ws.p : nullptr, wb, st);
    if (rc == METIS_OK) rc = metis_nvfp4_deferred_scales(parked.p, M, K, mode, dsc.p, du.p, st);
    HIP_OK(hipStreamSynchronize(st));
    std::vector<uint8_t> wc((size_t)(M * K / 2)), wsc((size_t)(M * K / 16));
    float wu = 0;
    metis_oracle_nvfp4_pack(x.data(), M, K, K, mode, nullptr, wc.data(), wsc.data(), &wu, nullptr);
    char line[200];
    snprintf(line, sizeof line, "metis_nvfp4_quant_project_deferred %lldx%lld r=%lld mode %d rc=%d: codes, scale bytes, unit bit-equal to the oracle",
             (long long)M, (long long)K, (long long)R, mode, rc);
    check(rc == METIS_OK && dc.download() == wc && dsc.download() == wsc && du.download()[0] == wu, line);
    const std::vector<uint16_t> gxv = dxv.download(), gt = dt.download();
    std::vector<double> got((size_t)(M * R)), want((size_t)(M * R));
    bool t_exact = true;
    for (int64_t m = 0; m < M; ++m)
        for (int64_t r = 0; r < R; ++r) {
            double acc = 0;
            for (int64_t k = 0; k < K; ++k) acc += (double)bf16_to_f32(x[(size_t)(m * K + k)]) * (double)bf16_to_f32(v[(size_t)(r * K + k)]);
            want[(size_t)(m * R + r)] = acc;
            got[(size_t)(m * R + r)] = bf16_to_f32(gxv[(size_t)(m * R + r)]);
            t_exact = t_exact && gt[(size_t)(m * R + r)] == metis_oracle_f32_to_bf16(bf16_to_f32(gxv[(size_t)(m * R + r)]) * bf16_to_f32(s[(size_t)r]));
        }
    snprintf(line, sizeof line, "  x V^T within one bf16 rounding of the double-precision product (%.2e), t = bf16(xv * s) exactly", rel_fro(got, want));
    check(rel_fro(got, want) <= 3e-3 && t_exact, line);
}

// Row- and column-blocked stochastic packings of one tensor from one pass: the bytes of the two separate calls.
static void check_sr_both(int64_t rows, int64_t cols, int mode, hipStream_t st)
{
    const std::vector<uint16_t> x = make_input(rows, cols, 11u, 1e-3f);
    DeviceBuffer<uint16_t> dx(x.size());
    dx.upload(x);
    const size_t nb = (size_t)(rows * cols / 16), wsb = metis_nvfp4_workspace_bytes(rows, cols);
    DeviceBuffer<uint8_t> cr(nb * 8), sr(nb), cc(nb * 8), sc(nb), cr2(nb * 8), sr2(nb), cc2(nb * 8), sc2(nb), ws(2 * wsb);
    DeviceBuffer<float> ur(1), uc(1), ur2(1), uc2(1);
    HIP_OK(hipMemset(ws.p, 0, 2 * wsb));
    const uint64_t seed = 0x1234567887654321ull, o_row = 17, o_col = (1ull << 35) + 3;
    int rc = metis_nvfp4_quant_sr_both(dx.p, rows, cols, cols, mode, seed, o_row, o_col, cr.p, sr.p, ur.p, cc.p, sc.p, uc.p, ws.p, 2 * wsb, st);
    if (rc == METIS_OK) rc = metis_nvfp4_quant_sr_row(dx.p, rows, cols, cols, mode, nullptr, seed, o_row, cr2.p, sr2.p, ur2.p, ws.p, wsb, st);
    if (rc == METIS_OK) rc = metis_nvfp4_quant_sr_col(dx.p, rows, cols, cols, mode, nullptr, seed, o_col, cc2.p, sc2.p, uc2.p, ws.p, wsb, st);
    HIP_OK(hipStreamSynchronize(st));
    char line[160];
    snprintf(line, sizeof line, "metis_nvfp4_quant_sr_both %lldx%lld mode %d rc=%d: both packings equal the separate calls", (long long)rows,
             (long long)cols, mode, rc);
    check(rc == METIS_OK && cr.download() == cr2.download() && sr.download() == sr2.download() && ur.download()[0] == ur2.download()[0] &&
              cc.download() == cc2.download() && sc.download() == sc2.download() && uc.download()[0] == uc2.download()[0], line);
}

int main()
{
    // before anything touches the GPU: this program and the library must agree on the layout of the member descriptors
    if (metis_linear_member_size() != sizeof(metis_linear_member)) {
        printf("FAIL: libmetis_hip.so was built with a metis_linear_member of %zu bytes, this program with %zu: rebuild it (make native-check)\n",
               metis_linear_member_size(), sizeof(metis_linear_member));
        return 1;
    }
    hipStream_t st;
    HIP_OK(hipStreamCreate(&st));                                // a caller-owned stream, default priority
    printf("library version %d\n", metis_version());

    // ---- 1 + 3: quantizer and dequantizer, both modes
    const int64_t rows = 96, cols = 512;
    const std::vector<uint16_t> x = make_input(rows, cols, 1u, 1.0f);
    for (int mode = 0; mode < 2; ++mode) {
        DeviceBuffer<uint8_t> dc((size_t)(rows * cols / 2)), ds((size_t)(rows * cols / 16));
        DeviceBuffer<float> du(1);
        const Packed got = quantize_on_device(x, rows, cols, mode, st, &dc, &ds, &du);
        Packed want;
        want.codes.resize(got.codes.size());
        want.scales.resize(got.scales.size());
        metis_oracle_nvfp4_pack(x.data(), rows, cols, cols, mode, nullptr, want.codes.data(), want.scales.data(), &want.unit, nullptr);
        check(got.codes == want.codes && got.scales == want.scales && got.unit == want.unit,
              mode == 0 ? "metis_nvfp4_quant_row P32: codes, scale bytes, unit bit-equal" : "metis_nvfp4_quant_row PB16: codes, scale bytes, unit bit-equal");
        DeviceBuffer<uint16_t> dout((size_t)(rows * cols));
        const int rc = metis_nvfp4_dequant(dc.p, ds.p, du.p, rows, cols, mode, dout.p, METIS_DTYPE_BF16, st);
        HIP_OK(hipStreamSynchronize(st));
        std::vector<uint16_t> want_dq((size_t)(rows * cols));
        metis_oracle_nvfp4_dequant(want.codes.data(), want.scales.data(), want.unit, rows, cols, mode, want_dq.data(), nullptr);
        std::vector<uint16_t> got_dq = dout.download();
        bool same = rc == METIS_OK;
        for (size_t i = 0; same && i < got_dq.size(); ++i)
            same = got_dq[i] == want_dq[i] || (bf16_to_f32(got_dq[i]) == 0.0f && bf16_to_f32(want_dq[i]) == 0.0f);
        check(same, mode == 0 ? "metis_nvfp4_dequant P32 -> bf16 bit-equal" : "metis_nvfp4_dequant PB16 -> bf16 bit-equal");
    }

    // ---- 2: fused RMSNorm -> quant
    {
        std::vector<uint16_t> gamma((size_t)cols);
        for (int64_t c = 0; c < cols; ++c) gamma[(size_t)c] = metis_oracle_f32_to_bf16(1.0f + 0.001f * (float)(c % 97));
        DeviceBuffer<uint16_t> dx(x.size()), dg(gamma.size()), dn(x.size());
        dx.upload(x);
        dg.upload(gamma);
        DeviceBuffer<uint8_t> dc((size_t)(rows * cols / 2)), ds((size_t)(rows * cols / 16));
        DeviceBuffer<float> du(1);
        const size_t wsb = metis_nvfp4_workspace_bytes(rows, cols);
        DeviceBuffer<uint8_t> ws(wsb);
        HIP_OK(hipMemset(ws.p, 0, wsb));
        const int rc = metis_rmsnorm_nvfp4_quant(dx.p, dg.p, 1e-6f, rows, cols, METIS_MODE_P32, dn.p, dc.p, ds.p, du.p, ws.p, wsb, st);
        HIP_OK(hipStreamSynchronize(st));
        std::vector<uint16_t> wn(x.size());
        std::vector<uint8_t> wc((size_t)(rows * cols / 2)), wsc((size_t)(rows * cols / 16));
        float wu = 0;
        metis_oracle_rmsnorm_nvfp4(x.data(), gamma.data(), 1e-6f, rows, cols, 0, wn.data(), wc.data(), wsc.data(), &wu);
        // the row sum of squares is accumulated in a different order on the device: compare the normed values
        // to one bf16 ulp and the packed tensor only where the normed values agree exactly
        const std::vector<uint16_t> gn = dn.download();
        size_t off_by_more = 0, differ = 0;
        for (size_t i = 0; i < gn.size(); ++i) {
            const int d = abs((int)gn[i] - (int)wn[i]);
            differ += d != 0;
            off_by_more += d > 1;
        }
        char line[160];
        snprintf(line, sizeof line, "metis_rmsnorm_nvfp4_quant rc=%d: normed within 1 bf16 ulp (%zu of %zu differ by 1)", rc, differ, gn.size());
        check(rc == METIS_OK && off_by_more == 0 && differ < gn.size() / 50, line);
        if (differ == 0) {
            check(dc.download() == wc && ds.download() == wsc && du.download()[0] == wu, "  packed tensor of the normed rows bit-equal");
        }
    }

    // ---- 4: GEMM, tiled and skinny dispatch
    check_linear(272, 320, 256, st, "tiled 256x256");
    check_linear(96, 132, 96, st, "tiled 128x128");
    check_linear(48, 160, 512, st, "skinny");

    // ---- 4b: the pipelined GEMM on tiled expansions, and the rotated quantizer
    check_tiled(272, 320, 256, st);
    check_tiled(512, 256, 2048, st);

    // ---- 6: split-K through a caller workspace
    check_linear(256, 256, 2048, st, "tiled, K split", true);
    check_linear(40, 64, 8192, st, "skinny, K split", true);

    // ---- 7 + 8: mean mode at decode size
    check_mean_mode_decode(st);
    check_decode_bf16(48, 160, 512, st);
    check_decode_bf16(64, 96, 8192, st);
    check_decode_rotated_weight(40, 96, 512, st);
    check_decode_three_launches(48, 160, 512, 32, st);
    check_decode_three_launches(64, 96, 4096, 64, st);

    // ---- 4b: one pass over an activation (quantizer + rank-r projection; K slices at 256 rows against a long K), and
    //          both stochastic packings of a gradient
    check_quant_project(288, 448, 32, METIS_MODE_P32, st);
    check_quant_project(256, 4096, 64, METIS_MODE_PB16, st);
    check_sr_both(272, 336, METIS_MODE_P32, st);
    check_sr_both(64, 1024, METIS_MODE_PB16, st);

    // ---- 5: error codes
    {
        DeviceBuffer<uint16_t> dx(1024);
        DeviceBuffer<uint8_t> dc(512), ds(64), ws(metis_nvfp4_workspace_bytes(32, 32));
        DeviceBuffer<float> du(1);
        check(metis_nvfp4_quant_row(dx.p, 32, 24, 24, 0, dc.p, ds.p, du.p, ws.p, ws.n, st) == METIS_E_SHAPE, "16 does not divide 24 -> METIS_E_SHAPE");
        check(metis_nvfp4_quant_row(dx.p, 32, 32, 32, 5, dc.p, ds.p, du.p, ws.p, ws.n, st) == METIS_E_ARG, "unknown mode -> METIS_E_ARG");
        check(metis_nvfp4_quant_row(dx.p, 32, 32, 32, 0, dc.p, ds.p, du.p, ws.p, 16, st) == METIS_E_WORKSPACE, "short workspace -> METIS_E_WORKSPACE");
        check(metis_nvfp4_quant_row(nullptr, 32, 32, 32, 0, dc.p, ds.p, du.p, ws.p, ws.n, st) == METIS_E_ARG, "null input -> METIS_E_ARG");
        check(metis_nvfp4_quant_row(nullptr, 0, 32, 32, 0, nullptr, nullptr, nullptr, nullptr, 0, st) == METIS_OK, "empty tensor is a no-op");
        check(strlen(metis_error_string(METIS_E_SHAPE)) > 0, "metis_error_string");
        // grouped entry: a split shape with a short workspace, a centre on a shape that cannot take one
        metis_linear_member one = {};
        DeviceBuffer<uint8_t> pa((size_t)(8 * 8192 / 2)), ps((size_t)(8 * 8192 / 16)), pb((size_t)(64 * 8192 / 2)), pbs((size_t)(64 * 8192 / 16));
        DeviceBuffer<float> un(1), o((size_t)(8 * 64)), cen(8192);
        one.b_codes = pb.p; one.b_scales = pbs.p; one.b_unit = un.p; one.out = o.p; one.N = 64;
        const size_t need = metis_linear_grouped_workspace_bytes(8, 8192, &one, 1);
        DeviceBuffer<uint8_t> gws(need + 16);
        check(need > 0 && metis_linear_fwd_grouped(pa.p, ps.p, un.p, 8, 8192, &one, 1, METIS_DTYPE_BF16, gws.p, 1024, st) == METIS_E_WORKSPACE,
              "grouped call, short split-K workspace -> METIS_E_WORKSPACE");
        check(metis_linear_fwd_grouped_centered(pa.p, ps.p, un.p, 8, 8192, &one, 1, METIS_DTYPE_BF16, nullptr, gws.p, need, st) == METIS_E_ARG,
              "centred call without a centre -> METIS_E_ARG");
        check(metis_linear_grouped_centered_supported(300, 8192, &one, 1, 1) == 0 &&
              metis_linear_fwd_grouped_centered(pa.p, ps.p, un.p, 300, 8192, &one, 1, METIS_DTYPE_BF16, cen.p, gws.p, need, st) == METIS_E_ARG,
              "centred call at M >= 256 -> not supported, METIS_E_ARG");
    }
    HIP_OK(hipStreamDestroy(st));
    printf(failures ? "FAILED %d check(s)\n" : "all checks passed\n", failures);
    return failures ? 1 : 0;
}
