/*
 * asan_main.c -- sanitizer driver of the CPU oracle (test infrastructure, like cpu_ref.c).
 *
 * Built by `make -C oracle asan` together with cpu_ref.c under -fsanitize=address,undefined.  Calls every
 * function of the oracle on heap buffers of exactly the size the call may touch (ragged shapes, every operand
 * layout, padded leading dimensions), so an access one element past a row or an operand is an AddressSanitizer
 * report, and checks each result against a plain loop written here.  Exit status 0 = clean.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

void ref_fill_uniform(float *, size_t, uint64_t, float, float);
void ref_fill_normal(float *, size_t, uint64_t);
void ref_fill_pattern(float *, size_t, int);
uint16_t ref_f32_to_bf16(float);
float ref_bf16_to_f32(uint16_t);
uint16_t ref_f32_to_f16(float);
float ref_f16_to_f32(uint16_t);
float ref_fp8_e4m3_to_f32(uint8_t);
uint8_t ref_f32_to_fp8_e4m3(float);
void ref_decode_fp8(const uint8_t *, float *, size_t);
void ref_encode_fp8(const float *, uint8_t *, size_t);
void ref_encode_bf16(const float *, uint16_t *, size_t);
void ref_decode_bf16(const uint16_t *, float *, size_t);
void ref_encode_f16(const float *, uint16_t *, size_t);
void ref_decode_f16(const uint16_t *, float *, size_t);
float ref_amax(const float *, size_t);
float ref_quantize_int8(const float *, int8_t *, size_t);
float ref_quantize_fp8(const float *, uint8_t *, size_t);
void ref_quantize_fp8_block(const float *, uint8_t *, float *, size_t, size_t, size_t, size_t);
void ref_quantize_int8_block(const float *, int8_t *, float *, size_t, size_t, size_t, size_t);
void ref_transpose(const void *, void *, size_t, size_t, size_t);
void ref_gemm_i8_i32(const int8_t *, size_t, size_t, const int8_t *, size_t, size_t, int32_t *, size_t, size_t, size_t, size_t);
void ref_scale_i32_to_f32(const int32_t *, float *, size_t, float, float);
void ref_gemm_f32acc(const float *, size_t, size_t, const float *, size_t, size_t, float *, size_t, size_t, size_t, size_t);
void ref_gemm_f64acc(const float *, size_t, size_t, const float *, size_t, size_t, double *, size_t, size_t, size_t, size_t);
void ref_gemm_fp8_block(const float *, size_t, size_t, const float *, size_t, size_t, const float *, size_t, size_t,
                        const float *, size_t, size_t, float *, size_t, size_t, size_t, size_t, size_t);
void ref_gemm_fp8_block_f64(const float *, size_t, size_t, const float *, size_t, size_t, const float *, size_t, size_t,
                            const float *, size_t, size_t, double *, size_t, size_t, size_t, size_t);
void ref_gemm_i8_block(const int8_t *, size_t, size_t, const int8_t *, size_t, size_t, const float *, size_t, size_t,
                       const float *, size_t, size_t, float *, size_t, size_t, size_t, size_t);
size_t ref_select_tile(size_t, int);
void ref_block_swizzle(size_t, size_t, size_t, size_t, size_t *, size_t *);
double ref_max_abs_diff(const float *, const float *, size_t);

static int failures = 0;
#define CHECK(cond)                                                          \
    do {                                                                     \
        if (!(cond)) {                                                       \
            fprintf(stderr, "%s:%d: check failed: %s\n", __FILE__, __LINE__, #cond); \
            ++failures;                                                      \
        }                                                                    \
    } while (0)

static void *xmalloc(size_t n) {
    void *p = malloc(n ? n : 1);
    if (!p) abort();
    return p;
}

/* element (m, k) of A and (n, k) of B under the three storages the oracle takes */
static void layout_strides(int layout, size_t M, size_t N, size_t K, size_t *a_rs, size_t *a_cs, size_t *b_ns, size_t *b_ks) {
    if (layout == 0) { *a_rs = K; *a_cs = 1; *b_ns = K; *b_ks = 1; }        /* nt */
    else if (layout == 1) { *a_rs = K; *a_cs = 1; *b_ns = 1; *b_ks = N; }   /* nn */
    else { *a_rs = 1; *a_cs = M; *b_ns = 1; *b_ks = N; }                    /* tn */
}

static void check_codecs(void) {
    /* every fp8 code survives a round trip; NaN codes decode to NaN */
    for (int b = 0; b < 256; ++b) {
        const float f = ref_fp8_e4m3_to_f32((uint8_t)b);
        if ((b & 0x7F) == 0x7F) CHECK(isnan(f));
        else CHECK(ref_f32_to_fp8_e4m3(f) == (uint8_t)b || f == 0.0f);
    }
    CHECK(ref_f32_to_fp8_e4m3(1e9f) == 0x7E && ref_f32_to_fp8_e4m3(-1e9f) == 0xFE);     /* saturate to 448 */
    const size_t n = 1003;
    float *x = xmalloc(n * 4), *y = xmalloc(n * 4);
    uint8_t *q8 = xmalloc(n);
    uint16_t *q16 = xmalloc(n * 2);
    ref_fill_normal(x, n, 7);
    ref_encode_fp8(x, q8, n);
    ref_decode_fp8(q8, y, n);
    for (size_t i = 0; i < n; ++i) CHECK(fabsf(y[i] - x[i]) <= 0.0625f * fabsf(x[i]) + 0.002f);
    ref_encode_bf16(x, q16, n);
    ref_decode_bf16(q16, y, n);
    for (size_t i = 0; i < n; ++i) CHECK(fabsf(y[i] - x[i]) <= 0.00391f * fabsf(x[i]) && ref_f32_to_bf16(y[i]) == q16[i]);
    ref_encode_f16(x, q16, n);
    ref_decode_f16(q16, y, n);
    for (size_t i = 0; i < n; ++i) CHECK(fabsf(y[i] - x[i]) <= 0.00049f * fabsf(x[i]) + 1e-7f && ref_f32_to_f16(y[i]) == q16[i]);
    CHECK(ref_f16_to_f32(ref_f32_to_f16(65504.0f)) == 65504.0f && ref_bf16_to_f32(ref_f32_to_bf16(-2.5f)) == -2.5f);
    ref_fill_uniform(x, n, 3, -1.0f, 1.0f);
    float amax = 0;
    for (size_t i = 0; i < n; ++i) { CHECK(x[i] >= -1.0f && x[i] <= 1.0f); amax = fmaxf(amax, fabsf(x[i])); }
    CHECK(ref_amax(x, n) == amax && ref_amax(x, 0) == 0.0f);
    ref_fill_pattern(x, n, 0);
    ref_fill_pattern(y, n, 1);
    free(x); free(y); free(q8); free(q16);
}

static void check_quantizers(void) {
    const size_t rows = 37, cols = 300, ld = 311;
    float *x = xmalloc(rows * ld * 4);
    ref_fill_normal(x, rows * ld, 11);
    int8_t *qi = xmalloc(rows * ld);
    const float si = ref_quantize_int8(x, qi, rows * ld);
    for (size_t i = 0; i < rows * ld; ++i) CHECK(fabsf(x[i] - si * (float)qi[i]) <= 0.5001f * si && qi[i] >= -127);
    uint8_t *qf = xmalloc(rows * ld);
    const float sf = ref_quantize_fp8(x, qf, rows * ld);
    CHECK(sf > 0 && si > 0);
    /* block quantiser: 1 x 128 and 128 x 128 blocks over a ragged matrix with a padded row stride */
    for (int square = 0; square < 2; ++square) {
        const size_t br = square ? 128 : 1, nbr = (rows + br - 1) / br, nbc = (cols + 127) / 128;
        float *xs = xmalloc(rows * cols * 4);
        for (size_t r = 0; r < rows; ++r) memcpy(xs + r * cols, x + r * ld, cols * 4);
        uint8_t *q = xmalloc(rows * cols);
        float *sc = xmalloc(nbr * nbc * 4);
        ref_quantize_fp8_block(xs, q, sc, rows, cols, br, 128);
        for (size_t r = 0; r < rows; ++r)
            for (size_t c = 0; c < cols; ++c) {
                const float s = sc[(r / br) * nbc + c / 128];
                CHECK(fabsf(xs[r * cols + c] - s * ref_fp8_e4m3_to_f32(q[r * cols + c])) <= 0.0626f * fabsf(xs[r * cols + c]) + 0.002f * s);
            }
        int8_t *q8 = xmalloc(rows * cols);
        ref_quantize_int8_block(xs, q8, sc, rows, cols, br, 128);
        for (size_t r = 0; r < rows; ++r)
            for (size_t c = 0; c < cols; ++c) {
                const float s = sc[(r / br) * nbc + c / 128];
                CHECK(fabsf(xs[r * cols + c] - s * (float)q8[r * cols + c]) <= 0.5001f * s);
            }
        free(xs); free(q); free(q8); free(sc);
    }
    free(x); free(qi); free(qf);
}

static void check_transpose(void) {
    static const size_t elems[] = {1, 2, 4};
    for (int e = 0; e < 3; ++e) {
        const size_t M = 45, N = 70, es = elems[e];
        uint8_t *in = xmalloc(M * N * es), *out = xmalloc(M * N * es), *back = xmalloc(M * N * es);
        for (size_t i = 0; i < M * N * es; ++i) in[i] = (uint8_t)(i * 31 + 7);
        ref_transpose(in, out, M, N, es);
        for (size_t m = 0; m < M; ++m)
            for (size_t n = 0; n < N; ++n) CHECK(memcmp(out + (n * M + m) * es, in + (m * N + n) * es, es) == 0);
        ref_transpose(out, back, N, M, es);
        CHECK(memcmp(back, in, M * N * es) == 0);
        free(in); free(out); free(back);
    }
}

static void check_gemms(void) {
    static const size_t shapes[][3] = {{1, 1, 1}, {5, 7, 13}, {33, 17, 128}, {16, 130, 300}, {40, 24, 257}};
    for (size_t si = 0; si < sizeof(shapes) / sizeof(shapes[0]); ++si)
        for (int layout = 0; layout < 3; ++layout) {
            const size_t M = shapes[si][0], N = shapes[si][1], K = shapes[si][2], ldc = N + 3;
            size_t a_rs, a_cs, b_ns, b_ks;
            layout_strides(layout, M, N, K, &a_rs, &a_cs, &b_ns, &b_ks);
            float *A = xmalloc(M * K * 4), *B = xmalloc(N * K * 4);
            int8_t *Ai = xmalloc(M * K), *Bi = xmalloc(N * K);
            ref_fill_uniform(A, M * K, 100 + si, -2.0f, 2.0f);
            ref_fill_uniform(B, N * K, 200 + si, -2.0f, 2.0f);
            for (size_t i = 0; i < M * K; ++i) { A[i] = rintf(A[i]); Ai[i] = (int8_t)(A[i] * 60.0f); }
            for (size_t i = 0; i < N * K; ++i) { B[i] = rintf(B[i]); Bi[i] = (int8_t)(B[i] * 60.0f); }
            int32_t *Ci = xmalloc(M * ldc * 4);
            float *Cf = xmalloc(M * ldc * 4), *Cs = xmalloc(M * ldc * 4);
            double *Cd = xmalloc(M * ldc * 8);
            for (size_t i = 0; i < M * ldc; ++i) { Ci[i] = -9; Cf[i] = -9.0f; Cd[i] = -9.0; }
            ref_gemm_i8_i32(Ai, a_rs, a_cs, Bi, b_ns, b_ks, Ci, ldc, M, N, K);
            ref_gemm_f32acc(A, a_rs, a_cs, B, b_ns, b_ks, Cf, ldc, M, N, K);
            ref_gemm_f64acc(A, a_rs, a_cs, B, b_ns, b_ks, Cd, ldc, M, N, K);
            ref_scale_i32_to_f32(Ci, Cs, M * ldc, 0.5f, 0.25f);
            for (size_t m = 0; m < M; ++m) {
                for (size_t n = 0; n < N; ++n) {
                    long long acc = 0;
                    double accd = 0;
                    for (size_t k = 0; k < K; ++k) {
                        acc += (long long)Ai[m * a_rs + k * a_cs] * Bi[n * b_ns + k * b_ks];
                        accd += (double)A[m * a_rs + k * a_cs] * B[n * b_ns + k * b_ks];
                    }
                    CHECK(Ci[m * ldc + n] == (int32_t)acc);
                    CHECK(Cd[m * ldc + n] == accd);                       /* small integers: exact in any order */
                    CHECK(Cf[m * ldc + n] == (float)accd);
                    CHECK(Cs[m * ldc + n] == (float)(int32_t)acc * 0.125f);
                }
                for (size_t n = N; n < ldc; ++n) CHECK(Ci[m * ldc + n] == -9 && Cf[m * ldc + n] == -9.0f && Cd[m * ldc + n] == -9.0);
            }
            CHECK(ref_max_abs_diff(Cf, Cf, M * ldc) == 0.0);
            /* block scales, both scale arrangements, the three K tiles of the reference's dispatch */
            const size_t KB = (K + 127) / 128, NB = (N + 127) / 128;
            float *as = xmalloc(M * KB * 4), *bs = xmalloc(NB * KB * 4);
            for (size_t i = 0; i < M * KB; ++i) as[i] = (float)(1 << (i % 3));
            for (size_t i = 0; i < NB * KB; ++i) bs[i] = 1.0f / (float)(1 << (i % 4));
            for (int col = 0; col < 2; ++col) {
                const size_t as_ms = col ? 1 : KB, as_ks = col ? M : 1, bs_ns = col ? 1 : KB, bs_ks = col ? NB : 1;
                static const size_t bks[] = {128, 64, 32};
                for (int t = 0; t < 3; ++t) {
                    for (size_t i = 0; i < M * ldc; ++i) { Cf[i] = -9.0f; Cd[i] = -9.0; }
                    ref_gemm_fp8_block(A, a_rs, a_cs, B, b_ns, b_ks, as, as_ms, as_ks, bs, bs_ns, bs_ks, Cf, ldc, M, N, K, bks[t]);
                    ref_gemm_fp8_block_f64(A, a_rs, a_cs, B, b_ns, b_ks, as, as_ms, as_ks, bs, bs_ns, bs_ks, Cd, ldc, M, N, K);
                    for (size_t m = 0; m < M; ++m)
                        for (size_t n = 0; n < N; ++n) {
                            double acc = 0;
                            for (size_t k = 0; k < K; ++k)
                                acc += (double)A[m * a_rs + k * a_cs] * B[n * b_ns + k * b_ks] * as[m * as_ms + (k / 128) * as_ks] *
                                       bs[(n / 128) * bs_ns + (k / 128) * bs_ks];
                            CHECK(Cd[m * ldc + n] == acc && Cf[m * ldc + n] == (float)acc);     /* powers of two: exact */
                        }
                }
                /* the int8 twin: exact int32 partial per K block, power-of-two scales: exact */
                for (size_t i = 0; i < M * ldc; ++i) Cf[i] = -9.0f;
                ref_gemm_i8_block(Ai, a_rs, a_cs, Bi, b_ns, b_ks, as, as_ms, as_ks, bs, bs_ns, bs_ks, Cf, ldc, M, N, K);
                for (size_t m = 0; m < M; ++m) {
                    for (size_t n = 0; n < N; ++n) {
                        double acc = 0;
                        for (size_t k = 0; k < K; ++k)
                            acc += (double)Ai[m * a_rs + k * a_cs] * Bi[n * b_ns + k * b_ks] * as[m * as_ms + (k / 128) * as_ks] *
                                   bs[(n / 128) * bs_ns + (k / 128) * bs_ks];
                        CHECK(Cf[m * ldc + n] == (float)acc);
                    }
                    for (size_t n = N; n < ldc; ++n) CHECK(Cf[m * ldc + n] == -9.0f);
                }
            }
            free(A); free(B); free(Ai); free(Bi); free(Ci); free(Cf); free(Cs); free(Cd); free(as); free(bs);
        }
}

static void check_tiles(void) {
    CHECK(ref_select_tile(6144, 0) == 128 && ref_select_tile(96, 1) == 32 && ref_select_tile(48, 2) == 0);
    const size_t tm_n = 7, tn_n = 5, group = 4;
    unsigned char seen[7 * 5];
    memset(seen, 0, sizeof seen);
    for (size_t b = 0; b < tm_n * tn_n; ++b) {
        size_t tm, tn;
        ref_block_swizzle(b, tm_n, tn_n, group, &tm, &tn);
        CHECK(tm < tm_n && tn < tn_n);
        if (tm < tm_n && tn < tn_n) seen[tm * tn_n + tn]++;
    }
    for (size_t i = 0; i < tm_n * tn_n; ++i) CHECK(seen[i] == 1);
}

int main(void) {
    check_codecs();
    check_quantizers();
    check_transpose();
    check_gemms();
    check_tiles();
    if (failures) {
        fprintf(stderr, "oracle_asan: %d check(s) failed\n", failures);
        return 1;
    }
    puts("oracle_asan: clean");
    return 0;
}
