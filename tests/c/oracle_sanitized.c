/* The CPU oracle compiled as one translation unit with AddressSanitizer and UndefinedBehaviorSanitizer and run over
 * every block format on random bytes (exact buffer sizes, so that a read or write one element past a block, a
 * row or an output shows), plus the dense, attention and decoder-glue functions.  Test infrastructure: built and run by
 * tests/test_oracle_sanitized.py only. */
#include "../../oracle/oracle.c"

#include <stdio.h>

static uint32_t rng_state = 12345u;
static uint32_t rnd(void) {
    rng_state = rng_state * 1664525u + 1013904223u;
    return rng_state >> 8;
}
static float rndf(void) { return (float)((int)(rnd() % 2001) - 1000) * 1e-3f; }

int main(void) {
    static const int types[] = {T_F32, T_F16, T_BF16, T_Q4_0, T_Q4_1, T_Q5_0, T_Q5_1, T_Q8_0, T_Q2_K, T_Q3_K, T_Q4_K,
                                T_Q5_K, T_Q6_K, T_Q8_K, T_IQ4_NL, T_IQ4_XS, T_TQ1_0, T_TQ2_0};
    const int n = 5, k = 768, m = 3;
    for (size_t ti = 0; ti < sizeof types / sizeof types[0]; ti++) {
        const int t = types[ti];
        int be, bb;
        if (orc_type_sizes(t, &be, &bb) != ORC_OK) { printf("type %d: no sizes\n", t); return 1; }
        if (orc_row_bytes(t, k) != (int64_t)k / be * bb) { printf("type %d: row bytes\n", t); return 1; }
        const size_t wbytes = (size_t)n * (k / be) * bb;
        uint8_t* w = (uint8_t*)malloc(wbytes);
        for (size_t i = 0; i < wbytes; i++) w[i] = (uint8_t)rnd();
        float* deq = (float*)malloc((size_t)n * k * sizeof(float));
        float* x = (float*)malloc((size_t)k * sizeof(float));
        float* y = (float*)malloc((size_t)n * sizeof(float));
        uint16_t* a = (uint16_t*)malloc((size_t)m * k * sizeof(uint16_t));
        float* c = (float*)malloc((size_t)m * n * sizeof(float));
        for (int i = 0; i < k; i++) x[i] = rndf();
        for (int i = 0; i < m * k; i++) a[i] = (uint16_t)(0x3c00u + (rnd() & 0x3ffu)) ; /* bf16 bit patterns of moderate size */
        if (orc_dequant(t, w, (int64_t)n * k, deq) != ORC_OK) { printf("type %d: dequant\n", t); return 1; }
        if (orc_matvec_q(t, w, n, k, x, y) != ORC_OK) { printf("type %d: matvec\n", t); return 1; }
        if (orc_matvec_q_reference_algorithm(t, w, n, k, x, y) != ORC_OK) { printf("type %d: reference matvec\n", t); return 1; }
        if (orc_gemm_q(t, w, n, k, a, m, c) != ORC_OK) { printf("type %d: gemm\n", t); return 1; }
        free(w), free(deq), free(x), free(y), free(a), free(c);
    }
    /* an unknown type and a row that is not a multiple of the block are refused, not read */
    {
        int be, bb;
        float out[4];
        uint8_t w[4] = {0, 0, 0, 0};
        if (orc_type_sizes(99, &be, &bb) == ORC_OK || orc_dequant(99, w, 4, out) == ORC_OK) { printf("unknown type accepted\n"); return 1; }
        if (orc_row_bytes(T_Q4_K, 100) >= 0) { printf("ragged row accepted\n"); return 1; }
    }
    /* dense reference semantics */
    {
        double xv[3] = {1, 2, 3}, B[6] = {1, 2, 3, 4, 5, 6}, yv[2], A[6] = {1, 2, 3, 4, 5, 6}, C[4];
        orc_dense_vecmat(xv, B, 3, 2, yv);
        orc_dense_matmul(A, B, 2, 3, 2, C);
        if (yv[0] != 22.0 || yv[1] != 28.0 || C[0] != 22.0 || C[3] != 64.0) { printf("dense\n"); return 1; }
    }
    /* attention over a flat cache, decoder glue */
    {
        const int n_seq = 2, n_head = 3, dim = 64, max_tokens = 7;
        int32_t n_ctx[2] = {7, 1};
        const size_t kv = (size_t)n_seq * max_tokens * n_head * dim;
        uint16_t* kk = (uint16_t*)malloc(kv * sizeof(uint16_t));
        uint16_t* vv = (uint16_t*)malloc(kv * sizeof(uint16_t));
        float* q = (float*)malloc((size_t)n_seq * n_head * dim * sizeof(float));
        float* o = (float*)malloc((size_t)n_seq * n_head * dim * sizeof(float));
        for (size_t i = 0; i < kv; i++) kk[i] = (uint16_t)(0x3800u + (rnd() & 0x3ffu)), vv[i] = (uint16_t)(0x3800u + (rnd() & 0x3ffu));
        for (int i = 0; i < n_seq * n_head * dim; i++) q[i] = rndf();
        orc_attn_decode(q, kk, vv, n_ctx, n_seq, n_head, dim, max_tokens, 0.125, o);
        float w[64], yv[64], g[64], u[64];
        for (int i = 0; i < 64; i++) w[i] = rndf(), g[i] = rndf(), u[i] = rndf();
        orc_rmsnorm(q, w, 64, 1e-5, yv);
        orc_rope(q, n_head, dim, 5, 10000.0);
        orc_swiglu(g, u, 64, yv);
        if (orc_argmax(yv, 64) < 0 || orc_argmax(yv, 64) >= 64) { printf("argmax\n"); return 1; }
        free(kk), free(vv), free(q), free(o);
    }
    printf("ok\n");
    return 0;
}
