/* A plain C99 client of include/skainet_hip.h: what a Kotlin/Native cinterop or Panama binding does, without
 * Python in between.  `abi_client host` exercises the entry points that need no device; `abi_client device`
 * runs one Q8_0 matvec whose answer is known in closed form and prints "ok". */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "skainet_hip.h"

#define CHECK(cond)                                                   \
    do {                                                              \
        if (!(cond)) {                                                \
            fprintf(stderr, "%s:%d: %s failed\n", __FILE__, __LINE__, #cond); \
            return 1;                                                 \
        }                                                             \
    } while (0)

static int host_leg(void) {
    int elems = 0, bytes = 0;
    CHECK(skn_abi_version() == 3);
    CHECK(skn_type_block(SKN_TYPE_Q4_K, &elems, &bytes) == SKN_OK && elems == 256 && bytes == 144);
    CHECK(skn_type_block(SKN_TYPE_Q8_0, &elems, &bytes) == SKN_OK && elems == 32 && bytes == 34);
    CHECK(skn_type_block(SKN_TYPE_Q6_K, &elems, &bytes) == SKN_OK && elems == 256 && bytes == 210);
    CHECK(skn_row_bytes(SKN_TYPE_Q4_K, 11008) == 6192);
    CHECK(skn_row_bytes(SKN_TYPE_Q4_K, 100) == SKN_ERR_SHAPE);
    CHECK(strstr(skn_last_error(NULL), "is not a multiple of block size (256)") != NULL);
    CHECK(strcmp(skn_status_string(SKN_ERR_POOL), skn_status_string(SKN_OK)) != 0);
    /* the library's seeded generators: the checksums tests/test_synth_abi.py holds for the same calls */
    {
        static uint8_t w[2 * 2 * 144];
        static float x[512];
        CHECK(skn_row_bytes(SKN_TYPE_Q4_K, 512) * 2 == (long long)sizeof w);
        CHECK(skn_synth_weight(SKN_TYPE_Q4_K, 2, 512, 42u, w, sizeof w) == SKN_OK);
        CHECK(skn_synth_checksum(w, sizeof w) == 0xB1D64B923C1648B4ull);
        CHECK(skn_synth_activation_f32(512, 42u, x) == SKN_OK);
        CHECK(skn_synth_checksum(x, sizeof x) == 0x9A9CFB33CCC7FEA4ull);
        CHECK(skn_synth_weight(SKN_TYPE_Q4_0, 2, 512, 42u, w, sizeof w) == SKN_ERR_TYPE);
    }
    return 0;
}

/* fp16 bit patterns of small powers of two */
static uint16_t half_pow2(int e) { return (uint16_t)((e + 15) << 10); }

static int device_leg(void) {
    enum { N = 6, K = 128, NB = K / 32 };
    skn_ctx* ctx = NULL;
    uint8_t w[N * NB * 34];
    float x[K], y[N], want[N];
    void *dw = NULL, *dx = NULL, *dy = NULL;
    int n, b, i;
    CHECK(skn_init(0, &ctx) == SKN_OK);
    /* row n, block b: d = 2^(b-2), quants i - 16 + n; x[k] = 1 for even k, -0.5 for odd k */
    for (i = 0; i < K; i++) x[i] = (i & 1) ? -0.5f : 1.0f;
    for (n = 0; n < N; n++) {
        double acc = 0.0;
        for (b = 0; b < NB; b++) {
            uint8_t* blk = w + (n * NB + b) * 34;
            const uint16_t d = half_pow2(b - 2);
            const double dv = (double)(1 << b) / 4.0;
            memcpy(blk, &d, 2);
            for (i = 0; i < 32; i++) {
                const int q = i - 16 + n;
                blk[2 + i] = (uint8_t)(int8_t)q;
                acc += dv * q * x[32 * b + i];
            }
        }
        want[n] = (float)acc;
    }
    CHECK(skn_malloc(ctx, sizeof w, &dw) == SKN_OK);
    CHECK(skn_malloc(ctx, sizeof x, &dx) == SKN_OK);
    CHECK(skn_malloc(ctx, sizeof y, &dy) == SKN_OK);
    CHECK(skn_upload(ctx, dw, w, sizeof w) == SKN_OK);
    CHECK(skn_upload(ctx, dx, x, sizeof x) == SKN_OK);
    CHECK(skn_matvec_q(ctx, SKN_TYPE_Q8_0, dw, N, K, (const float*)dx, (float*)dy) == SKN_OK);
    CHECK(skn_download(ctx, y, dy, sizeof y) == SKN_OK);
    for (n = 0; n < N; n++) CHECK(y[n] == want[n]); /* every term is exact in fp32 */
    CHECK(skn_matvec_q(ctx, SKN_TYPE_Q8_0, dw, N, 100, (const float*)dx, (float*)dy) == SKN_ERR_SHAPE);
    CHECK(strstr(skn_last_error(ctx), "block size (32)") != NULL);
    CHECK(skn_free(ctx, dw) == SKN_OK && skn_free(ctx, dx) == SKN_OK && skn_free(ctx, dy) == SKN_OK);
    skn_shutdown(ctx);
    return 0;
}

int main(int argc, char** argv) {
    const int rc = (argc > 1 && strcmp(argv[1], "device") == 0) ? device_leg() : host_leg();
    if (rc == 0) puts("ok");
    return rc;
}
