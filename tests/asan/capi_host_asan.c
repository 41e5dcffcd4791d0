/*
 * capi_host_asan.c -- sanitizer driver of the host side of the C ABI (include/qgemm.h).
 *
 * Linked against a build of libqgemm.so whose host code is compiled under AddressSanitizer and
 * UndefinedBehaviorSanitizer (`make -C qgemm_amd/csrc asan`), and sanitized itself.  Walks the code that runs
 * before any kernel is launched and needs no GPU: argument validation of every entry point, status strings, the
 * tile raster, the option table, and above all the planner (qgemm_plan: cost estimate, K split, row split, choice
 * of the scale arrangement) over a sweep of shapes, types and storages.  Exit status 0 = clean.
 */
#include <stdio.h>
#include <string.h>

#include "qgemm.h"

static int failures = 0;
#define CHECK(cond)                                                          \
    do {                                                                     \
        if (!(cond)) {                                                       \
            fprintf(stderr, "%s:%d: check failed: %s\n", __FILE__, __LINE__, #cond); \
            ++failures;                                                      \
        }                                                                    \
    } while (0)

int main(void) {
    char buf[160], tiny[4];
    void *p = (void *)(size_t)4096;        /* never dereferenced: the calls below fail before any device access */
    const int have_gpu = qgemm_device_count() > 0;

    for (int st = -2; st < 16; ++st) CHECK(qgemm_status_string(st) != NULL && strlen(qgemm_status_string(st)) > 0);

    /* planner: every type and scale mode, square / oblong / skinny / huge shapes, the four storages */
    static const size_t dims[] = {1, 16, 100, 128, 256, 1000, 1024, 2048, 4608, 6144, 7168, 8192, 28672};
    static const int types[] = {QGEMM_DT_I8, QGEMM_DT_F8E4M3, QGEMM_DT_BF16, QGEMM_DT_F16};
    const size_t nd = sizeof(dims) / sizeof(dims[0]);
    long planned = 0;
    for (int t = 0; t < 4; ++t)
        for (int mode = 0; mode <= 2; ++mode)
            for (int km = 0; km <= 3; ++km)
                for (size_t i = 0; i < nd; ++i)
                    for (size_t j = 0; j < nd; j += 2)
                        for (size_t k = 1; k < nd; k += 3) {
                            const int st = qgemm_plan(types[t], mode, km, dims[i], dims[j], dims[k], buf, sizeof buf);
                            CHECK(st == QGEMM_OK || st == QGEMM_ERR_UNSUPPORTED || st == QGEMM_ERR_TOO_LARGE);
                            if (st == QGEMM_OK) { CHECK(strlen(buf) > 0 && strlen(buf) < sizeof buf); ++planned; }
                        }
    CHECK(planned > 1000);
    CHECK(qgemm_plan(QGEMM_DT_F8E4M3, QGEMM_SCALE_BLOCK128, 0, 6144, 4608, 7168, tiny, sizeof tiny) == QGEMM_OK && strlen(tiny) == 3);
    CHECK(qgemm_plan(QGEMM_DT_F8E4M3, QGEMM_SCALE_PER_MATRIX, 0, (size_t)1 << 22, (size_t)1 << 22, 128, buf, sizeof buf) == QGEMM_ERR_TOO_LARGE);
    CHECK(qgemm_plan(QGEMM_DT_F8E4M3, 1, 0, 0, 1, 1, buf, sizeof buf) == QGEMM_ERR_INVALID_ARG);
    CHECK(qgemm_plan(QGEMM_DT_F8E4M3, 1, 0, 1, 1, 1, NULL, 0) == QGEMM_ERR_INVALID_ARG);
    CHECK(qgemm_plan(99, 1, 0, 1, 1, 1, buf, sizeof buf) == QGEMM_ERR_UNSUPPORTED);
    /* forced rows (by name, every row of the two families below) and splits through the option table */
    {
        const int nb = qgemm_variant_count(QGEMM_DT_F8E4M3, QGEMM_SCALE_BLOCK128, 0);
        const int ni = qgemm_variant_count(QGEMM_DT_I8, QGEMM_SCALE_PER_MATRIX, 0);
        CHECK(nb > 4 && ni > 4 && qgemm_variant_count(99, 1, 0) == 0 && qgemm_variant_count(QGEMM_DT_BF16, QGEMM_SCALE_BLOCK128, 0) == 0);
        CHECK(qgemm_variant_name(QGEMM_DT_I8, 1, 0, ni, buf, sizeof buf) == QGEMM_ERR_INVALID_ARG);
        CHECK(qgemm_variant_name(QGEMM_DT_I8, 1, 0, 0, NULL, 0) == QGEMM_ERR_INVALID_ARG);
        for (int v = 0; v < nb + ni; ++v) {
            char name[64], other[64];
            const int blockfam = v < nb;
            CHECK(qgemm_variant_name(blockfam ? QGEMM_DT_F8E4M3 : QGEMM_DT_I8, blockfam ? QGEMM_SCALE_BLOCK128 : QGEMM_SCALE_PER_MATRIX,
                                     0, blockfam ? v : v - nb, name, sizeof name) == QGEMM_OK && strlen(name) > 0);
            CHECK(qgemm_force_config(name) == QGEMM_OK);
            for (long sp = 0; sp <= 4; ++sp) {
                CHECK(qgemm_set_option("force_split", sp) == QGEMM_OK);
                /* a family without a row of that name refuses, the one that has it plans it */
                int st = qgemm_plan(QGEMM_DT_F8E4M3, QGEMM_SCALE_BLOCK128, 0, 300, 520, 1280, buf, sizeof buf);
                CHECK(st == QGEMM_OK || st == QGEMM_ERR_UNSUPPORTED);
                if (blockfam) CHECK(st == QGEMM_OK && strlen(buf) >= 3);      /* (the name may be the row's twin for the other a_scale arrangement) */
                st = qgemm_plan(QGEMM_DT_I8, QGEMM_SCALE_PER_MATRIX, 0, 64, 7168, 2048, other, sizeof other);
                CHECK(st == QGEMM_OK || st == QGEMM_ERR_UNSUPPORTED);
                if (!blockfam) CHECK(st == QGEMM_OK && strncmp(other, name, strlen(name)) == 0);
            }
        }
        CHECK(qgemm_force_config("no_such_row") == QGEMM_ERR_INVALID_ARG);
        CHECK(qgemm_set_option("force_config", 3) == QGEMM_ERR_INVALID_ARG);
        CHECK(qgemm_force_config(NULL) == QGEMM_OK && qgemm_force_config("") == QGEMM_OK);
    }
    CHECK(qgemm_set_option("force_config", -1) == QGEMM_OK && qgemm_set_option("force_split", 0) == QGEMM_OK);
    CHECK(qgemm_set_option("no_such_option", 1) == QGEMM_ERR_INVALID_ARG && qgemm_set_option(NULL, 1) == QGEMM_ERR_INVALID_ARG);
    CHECK(qgemm_last_config(buf, sizeof buf) == QGEMM_OK && qgemm_last_config(NULL, 0) == QGEMM_ERR_INVALID_ARG);

    /* tile raster: a bijection for every group size, and the range check */
    for (uint32_t tm = 1; tm <= 9; ++tm)
        for (uint32_t tn = 1; tn <= 11; tn += 2)
            for (uint32_t g = 0; g <= 16; g += 4) {
                unsigned char seen[9 * 11];
                memset(seen, 0, sizeof seen);
                for (uint32_t w = 0; w < tm * tn; ++w) {
                    uint32_t a = 0, b = 0;
                    CHECK(qgemm_tile_map(w, tm, tn, g, &a, &b) == QGEMM_OK && a < tm && b < tn);
                    if (a < tm && b < tn) seen[a * tn + b]++;
                }
                for (uint32_t i = 0; i < tm * tn; ++i) CHECK(seen[i] == 1);
                uint32_t a, b;
                CHECK(qgemm_tile_map(tm * tn, tm, tn, g, &a, &b) == QGEMM_ERR_INVALID_ARG);
            }

    /* argument validation in front of the device */
    CHECK(qgemm_gemm(99, 0, 1, p, 16, p, 16, p, 16, 16, 16, 16, NULL) == QGEMM_ERR_UNSUPPORTED);
    CHECK(qgemm_gemm(QGEMM_DT_BF16, QGEMM_DT_F32, 7, p, 16, p, 16, p, 16, 16, 16, 16, NULL) == QGEMM_ERR_INVALID_ARG);
    CHECK(qgemm_gemm(QGEMM_DT_BF16, QGEMM_DT_F32, 1, p, 8, p, 16, p, 16, 16, 16, 16, NULL) == QGEMM_ERR_INVALID_ARG);
    CHECK(qgemm_gemm(QGEMM_DT_BF16, QGEMM_DT_F32, 1, p, 16, p, 16, p, 16, 0, 16, 16, NULL) == QGEMM_OK);
    CHECK(qgemm_scaled_gemm(QGEMM_DT_F8E4M3, QGEMM_DT_BF16, 2, 1, p, p, NULL, NULL, p, 64, 48, 64, 128, 0, NULL) == QGEMM_ERR_NOT_DIVISIBLE_M);
    CHECK(qgemm_scaled_gemm(QGEMM_DT_F8E4M3, QGEMM_DT_BF16, 2, 0, p, p, NULL, NULL, p, 64, 64, 64, 128, 0, NULL) == QGEMM_ERR_INVALID_ARG);
    CHECK(qgemm_scaled_gemm_static(QGEMM_DT_I8, QGEMM_DT_I32, 2, 0, p, p, p, p, p, 64, 64, 64, 128, 0, NULL) == QGEMM_ERR_UNSUPPORTED);
    CHECK(qgemm_transpose(3, p, p, 4, 4, NULL) == QGEMM_ERR_UNSUPPORTED);
    CHECK(qgemm_transpose(2, p, p, (size_t)1 << 31, 4, NULL) == QGEMM_ERR_TOO_LARGE);
    CHECK(qgemm_quantize(QGEMM_DT_I8, QGEMM_DT_I8, 1, p, 4, 4, 4, p, 4, (float *)p, 0, 0, NULL) == QGEMM_ERR_UNSUPPORTED);
    CHECK(qgemm_quantize(QGEMM_DT_F32, QGEMM_DT_F32, 2, p, 4, 4, 4, p, 4, (float *)p, 0, 0, NULL) == QGEMM_ERR_UNSUPPORTED);
    void *base = p;
    size_t bytes = 7;
    CHECK(qgemm_workspace_info(&base, &bytes) == QGEMM_OK && qgemm_workspace_info(NULL, NULL) == QGEMM_ERR_INVALID_ARG);
    if (!have_gpu) {
        CHECK(base == NULL && bytes == 0);
        CHECK(qgemm_init() == QGEMM_ERR_NO_DEVICE);
        CHECK(qgemm_reserve_workspace(1 << 20) == QGEMM_ERR_NO_DEVICE);
        CHECK(qgemm_gemm(QGEMM_DT_BF16, QGEMM_DT_F32, 1, p, 16, p, 16, p, 16, 16, 16, 16, NULL) == QGEMM_ERR_NO_DEVICE);
        CHECK(qgemm_selftest_layouts(buf, sizeof buf) == QGEMM_ERR_NO_DEVICE);
    }
    CHECK(qgemm_shutdown() == QGEMM_OK);
    if (failures) {
        fprintf(stderr, "capi_host_asan: %d check(s) failed\n", failures);
        return 1;
    }
    puts("capi_host_asan: clean");
    return 0;
}
