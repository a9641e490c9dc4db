/*
 * CPU oracle for the quantized-inference hot path.  TEST INFRASTRUCTURE ONLY:
 * this file is the checker that the HIP library is compared against (and the
 * "port" CPU baseline that the bench times next to the GPU figure).  Nothing in
 * the product path links, loads or calls it.
 *
 * What it restates, and where each piece comes from:
 *   - block sizes / type ids ......... reference gguf/src/commonMain/kotlin/sk/ai/net/gguf/Constants.kt:14-52,55,58-90
 *   - row -> byte-row rule ........... reference gguf/src/commonMain/kotlin/sk/ai/net/gguf/Quants.kt:10-20
 *   - element count / byte count ..... reference gguf/src/commonMain/kotlin/sk/ai/net/gguf/GGUFReader.kt:354-360
 *   - dense vec x mat, mat x mat ..... reference core/src/commonMain/kotlin/sk/ai/net/impl/DoublesTensor.kt:255-264,267-279
 *   - Linear = x . W^T + b ........... reference core/src/commonMain/kotlin/sk/ai/net/nn/Linear.kt:43-49
 *   - Q8_0 / Q4_K / Q6_K bit packing . NOT in the reference (Quants.kt:8 is a TODO).  The reference names its
 *     source as llama.cpp's gguf-py (Quants.kt:4-5, Constants.kt:4-5) without pinning a version; the packing
 *     below is the published ggml block definition (block_q8_0, block_q4_K with get_scale_min_k4, block_q6_K).
 *
 * Parity status per function (what pins it besides this file):
 *   orc_type_sizes, orc_row_bytes ..... pinned by the reference table itself (tests compare the literal numbers)
 *   orc_dense_vecmat, orc_dense_matmul pinned by the reference's TensorTest known answers (tests/golden/tensor_test_vectors.json)
 *   orc_dequant_* ..................... unpinned by the reference (it has no dequantizer); pinned by hand-built
 *                                       single-block known answers, an independent NumPy restatement
 *                                       (oracle/oracle_np.py) and the fp64 closed form rounded once
 *   deq_q4_0 ... deq_tq2_0 ............ the further formats of the reference's size table: unpinned by the reference
 *                                       in the same way; pinned by hand-built tagged blocks (element order, fifth-bit
 *                                       positions, scale indices), the NumPy restatement and exact rational goldens
 *                                       (tests/golden/quant_blocks_more.npz)
 *   orc_matvec_q / orc_gemm_q ......... pinned by reduction to the dense reference semantics on dequantized weights
 *   orc_attn_decode ................... unpinned by the reference (its softmax is not max-subtracted and is untested);
 *                                       pinned by closed forms (uniform K => mean(V), one token => V0) and scipy softmax
 *   orc_rmsnorm / orc_rope / orc_swiglu / orc_argmax: unpinned by the reference (absent there); closed forms only
 *
 * Build: see oracle/Makefile  (gcc -O3 -ffp-contract=off -fopenmp -shared -fPIC).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_OK 0
#define ORC_ERR_TYPE (-2)
#define ORC_ERR_SHAPE (-3)

enum { T_F32 = 0, T_F16 = 1, T_Q4_0 = 2, T_Q4_1 = 3, T_Q5_0 = 6, T_Q5_1 = 7, T_Q8_0 = 8, T_Q2_K = 10, T_Q4_K = 12,
       T_Q5_K = 13, T_Q6_K = 14, T_BF16 = 30, T_Q3_K = 11, T_Q8_K = 15, T_IQ4_NL = 20, T_IQ4_XS = 23, T_TQ1_0 = 34, T_TQ2_0 = 35 };

/* ---------------------------------------------------------------- scalars */

/* IEEE binary16 -> binary32, subnormals honoured. */
float orc_h2f(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: value = man * 2^-24 */
            float f = (float)man * 5.9604644775390625e-08f;
            memcpy(&bits, &f, 4);
            bits |= sign;
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float out;
    memcpy(&out, &bits, 4);
    return out;
}

/* binary32 -> binary16, round to nearest even. */
uint16_t orc_f2h(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7FFFFFFFu;
    if (ax >= 0x7F800000u) { /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | ((ax > 0x7F800000u) ? 0x200u : 0));
    }
    if (ax >= 0x477FF000u) { /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7C00u);
    }
    if (ax < 0x33000001u) { /* < 2^-25 (or exactly 2^-25 -> ties to even 0) */
        return (uint16_t)sign;
    }
    int32_t e = (int32_t)(ax >> 23) - 127;
    uint32_t m = (ax & 0x7FFFFFu) | 0x800000u;
    uint32_t shift, hm;
    if (e < -14) { /* subnormal half */
        shift = (uint32_t)(13 + (-14 - e));
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        hm = m >> shift;
        if (rem > half || (rem == half && (hm & 1u))) hm++;
        return (uint16_t)(sign | hm);
    }
    shift = 13;
    uint32_t rem = m & 0x1FFFu;
    hm = ((uint32_t)(e + 15) << 10) | ((m >> 13) & 0x3FFu);
    if (rem > 0x1000u || (rem == 0x1000u && (hm & 1u))) hm++;
    return (uint16_t)(sign | hm);
}

float orc_bf2f(uint16_t b) {
    uint32_t bits = (uint32_t)b << 16;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t orc_f2bf(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((x >> 16) | 0x40u);
    uint32_t lsb = (x >> 16) & 1u;
    x += 0x7FFFu + lsb;
    return (uint16_t)(x >> 16);
}

void orc_h2f_n(const uint16_t* h, float* f, int64_t n) {
    for (int64_t i = 0; i < n; i++) f[i] = orc_h2f(h[i]);
}
void orc_f2h_n(const float* f, uint16_t* h, int64_t n) {
    for (int64_t i = 0; i < n; i++) h[i] = orc_f2h(f[i]);
}

/* ------------------------------------------------------ type table / shapes */

/* Constants.kt:58-90 (the types this library computes with). */
int orc_type_sizes(int type, int* block_elems, int* block_bytes) {
    switch (type) {
        case T_F32: *block_elems = 1; *block_bytes = 4; return ORC_OK;
        case T_F16: *block_elems = 1; *block_bytes = 2; return ORC_OK;
        case T_BF16: *block_elems = 1; *block_bytes = 2; return ORC_OK;
        case T_Q4_0: *block_elems = 32; *block_bytes = 2 + 16; return ORC_OK;
        case T_Q4_1: *block_elems = 32; *block_bytes = 2 + 2 + 16; return ORC_OK;
        case T_Q5_0: *block_elems = 32; *block_bytes = 2 + 4 + 16; return ORC_OK;
        case T_Q5_1: *block_elems = 32; *block_bytes = 2 + 2 + 4 + 16; return ORC_OK;
        case T_Q2_K: *block_elems = 256; *block_bytes = 2 + 2 + 256 / 16 + 256 / 4; return ORC_OK;
        case T_Q5_K: *block_elems = 256; *block_bytes = 2 + 2 + 256 / 2 + 256 / 8 + 12; return ORC_OK;
        case T_Q3_K: *block_elems = 256; *block_bytes = 2 + 256 / 4 + 256 / 8 + 12; return ORC_OK;
        case T_Q8_K: *block_elems = 256; *block_bytes = 4 + 256 + 256 / 8; return ORC_OK;
        case T_IQ4_NL: *block_elems = 32; *block_bytes = 2 + 16; return ORC_OK;
        case T_IQ4_XS: *block_elems = 256; *block_bytes = 2 + 2 + 256 / 2 + 256 / 64; return ORC_OK;
        case T_TQ1_0: *block_elems = 256; *block_bytes = 2 + 4 * 13; return ORC_OK;
        case T_TQ2_0: *block_elems = 256; *block_bytes = 2 + 64; return ORC_OK;
        case T_Q8_0: *block_elems = 32; *block_bytes = 2 + 32; return ORC_OK;
        case T_Q4_K: *block_elems = 256; *block_bytes = 2 + 2 + 256 / 2 + 12; return ORC_OK;
        case T_Q6_K: *block_elems = 256; *block_bytes = 2 + 256 / 2 + 256 / 4 + 256 / 16; return ORC_OK;
        default: return ORC_ERR_TYPE;
    }
}

/* Quants.kt:10-20: last dim K -> K / block * bytes; K must be a block multiple. */
int64_t orc_row_bytes(int type, int64_t K) {
    int be, bb;
    if (orc_type_sizes(type, &be, &bb) != ORC_OK) return ORC_ERR_TYPE;
    if (K < 0 || K % be != 0) return ORC_ERR_SHAPE;
    return K / be * bb;
}

/* --------------------------------------------------------------- dequant */

/* Q8_0: d f16 @0, qs i8[32] @2.  y = d * q. */
static void deq_q8_0_block(const uint8_t* b, float* y) {
    uint16_t dh;
    memcpy(&dh, b, 2);
    const float d = orc_h2f(dh);
    const int8_t* qs = (const int8_t*)(b + 2);
    for (int i = 0; i < 32; i++) y[i] = d * (float)qs[i];
}

/* 6-bit scale / min of sub-block j out of the 12 packed bytes. */
static void q4k_scale_min(int j, const uint8_t* s, int* sc, int* m) {
    if (j < 4) {
        *sc = s[j] & 63;
        *m = s[j + 4] & 63;
    } else {
        *sc = (s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4);
        *m = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
    }
}

/* Q4_K: d f16 @0, dmin f16 @2, scales u8[12] @4, qs u8[128] @16.  Element-indexed form. */
static void deq_q4_k_block(const uint8_t* b, float* y) {
    uint16_t dh, mh;
    memcpy(&dh, b, 2);
    memcpy(&mh, b + 2, 2);
    const float d = orc_h2f(dh), dmin = orc_h2f(mh);
    const uint8_t* scales = b + 4;
    const uint8_t* qs = b + 16;
    for (int e = 0; e < 256; e++) {
        int c = e / 64, r = e % 64;
        int j = 2 * c + (r >= 32);
        int sc, m;
        q4k_scale_min(j, scales, &sc, &m);
        uint8_t byte = qs[32 * c + (r % 32)];
        int q = (r < 32) ? (byte & 0x0F) : (byte >> 4);
        float d1 = d * (float)sc;
        float m1 = dmin * (float)m;
        y[e] = d1 * (float)q - m1;
    }
}

/* Q6_K: ql u8[128] @0, qh u8[64] @128, scales i8[16] @192, d f16 @208. */
static void deq_q6_k_block(const uint8_t* b, float* y) {
    const uint8_t* ql = b;
    const uint8_t* qh = b + 128;
    const int8_t* sc = (const int8_t*)(b + 192);
    uint16_t dh;
    memcpy(&dh, b + 208, 2);
    const float d = orc_h2f(dh);
    for (int n = 0; n < 2; n++) {
        const uint8_t* qlp = ql + 64 * n;
        const uint8_t* qhp = qh + 32 * n;
        const int8_t* scp = sc + 8 * n;
        float* yp = y + 128 * n;
        for (int l = 0; l < 32; l++) {
            int is = l / 16;
            int q1 = (int)((qlp[l] & 0x0F) | (((qhp[l] >> 0) & 3) << 4)) - 32;
            int q2 = (int)((qlp[l + 32] & 0x0F) | (((qhp[l] >> 2) & 3) << 4)) - 32;
            int q3 = (int)((qlp[l] >> 4) | (((qhp[l] >> 4) & 3) << 4)) - 32;
            int q4 = (int)((qlp[l + 32] >> 4) | (((qhp[l] >> 6) & 3) << 4)) - 32;
            yp[l + 0] = d * (float)scp[is + 0] * (float)q1;
            yp[l + 32] = d * (float)scp[is + 2] * (float)q2;
            yp[l + 64] = d * (float)scp[is + 4] * (float)q3;
            yp[l + 96] = d * (float)scp[is + 6] * (float)q4;
        }
    }
}

/* ---- the other block formats of the reference's table (Constants.kt:58-90) that this library computes with.
 * Their packing is the published ggml definition as well (block_q4_0/q4_1/q5_0/q5_1/q2_K/q5_K); like the three
 * above they are unpinned by the reference.  Each value is an exact real (products of an f16 with small
 * integers) rounded once, so the fp32 order of operations below is immaterial. */

static float rd_h(const uint8_t* p) {
    uint16_t h;
    memcpy(&h, p, 2);
    return orc_h2f(h);
}

/* Q4_0: d f16 @0, qs u8[16] @2.  Low nibbles are elements 0..15, high nibbles 16..31; y = d * (q - 8). */
static void deq_q4_0_block(const uint8_t* b, float* y) {
    const float d = rd_h(b);
    for (int j = 0; j < 16; j++) {
        y[j] = d * (float)((int)(b[2 + j] & 0x0F) - 8);
        y[j + 16] = d * (float)((int)(b[2 + j] >> 4) - 8);
    }
}

/* Q4_1: d f16 @0, m f16 @2, qs u8[16] @4.  y = d * q + m. */
static void deq_q4_1_block(const uint8_t* b, float* y) {
    const float d = rd_h(b), m = rd_h(b + 2);
    for (int j = 0; j < 16; j++) {
        y[j] = d * (float)(b[4 + j] & 0x0F) + m;
        y[j + 16] = d * (float)(b[4 + j] >> 4) + m;
    }
}

/* Q5_0: d f16 @0, qh u32 @2 (bit j = fifth bit of element j), qs u8[16] @6.  y = d * (q - 16). */
static void deq_q5_0_block(const uint8_t* b, float* y) {
    const float d = rd_h(b);
    uint32_t qh;
    memcpy(&qh, b + 2, 4);
    for (int j = 0; j < 16; j++) {
        const int lo = (b[6 + j] & 0x0F) | (int)(((qh >> j) & 1u) << 4);
        const int hi = (b[6 + j] >> 4) | (int)(((qh >> (j + 16)) & 1u) << 4);
        y[j] = d * (float)(lo - 16);
        y[j + 16] = d * (float)(hi - 16);
    }
}

/* Q5_1: d f16 @0, m f16 @2, qh u32 @4, qs u8[16] @8.  y = d * q + m. */
static void deq_q5_1_block(const uint8_t* b, float* y) {
    const float d = rd_h(b), m = rd_h(b + 2);
    uint32_t qh;
    memcpy(&qh, b + 4, 4);
    for (int j = 0; j < 16; j++) {
        const int lo = (b[8 + j] & 0x0F) | (int)(((qh >> j) & 1u) << 4);
        const int hi = (b[8 + j] >> 4) | (int)(((qh >> (j + 16)) & 1u) << 4);
        y[j] = d * (float)lo + m;
        y[j + 16] = d * (float)hi + m;
    }
}

/* Q2_K: scales u8[16] @0 (low nibble scale, high nibble min), qs u8[64] @16, d f16 @80, dmin f16 @82.
 * Element e: half n = e / 128, bit pair j = (e % 128) / 32, l = e % 32: byte qs[32n + l] >> 2j, scale
 * 8n + 2j + (l >= 16).  y = (d * sc) * q - dmin * m. */
static void deq_q2_k_block(const uint8_t* b, float* y) {
    const float d = rd_h(b + 80), dmin = rd_h(b + 82);
    for (int e = 0; e < 256; e++) {
        const int n = e / 128, j = (e % 128) / 32, l = e % 32;
        const uint8_t s = b[8 * n + 2 * j + (l >= 16)];
        const int q = (b[16 + 32 * n + l] >> (2 * j)) & 3;
        y[e] = d * (float)(s & 0x0F) * (float)q - dmin * (float)(s >> 4);
    }
}

/* Q5_K: d f16 @0, dmin f16 @2, scales u8[12] @4 (as Q4_K), qh u8[32] @16, qs u8[128] @48.  Element e: chunk
 * c = e / 64, r = e % 64, sub-block 2c + (r >= 32), nibble of qs[32c + r % 32] (low for r < 32), fifth bit =
 * bit 2c + (r >= 32) of qh[r % 32].  y = (d * sc) * q - dmin * m. */
static void deq_q5_k_block(const uint8_t* b, float* y) {
    const float d = rd_h(b), dmin = rd_h(b + 2);
    for (int e = 0; e < 256; e++) {
        const int c = e / 64, r = e % 64, up = r >= 32;
        int sc, m;
        q4k_scale_min(2 * c + up, b + 4, &sc, &m);
        const uint8_t byte = b[48 + 32 * c + (r % 32)];
        const int q = (up ? byte >> 4 : byte & 0x0F) | (((b[16 + (r % 32)] >> (2 * c + up)) & 1) << 4);
        y[e] = d * (float)sc * (float)q - dmin * (float)m;
    }
}

/* Q3_K: hmask u8[32] @0, qs u8[64] @32, scales u8[12] @96, d f16 @108.  Sixteen 6-bit scales (low nibbles of
 * bytes 0..7 for scales 0..7, high nibbles for 8..15; two more bits each from bytes 8..11), stored with an
 * offset of 32.  Element e: half n = e / 128, bit pair j = (e % 128) / 32, l = e % 32: two bits of qs[32n + l] at
 * 2j, minus 4 unless bit 4n + j of hmask[l] is set; scale 8n + 2j + (l >= 16).  y = d * (sc - 32) * q. */
static void deq_q3_k_block(const uint8_t* b, float* y) {
    const float d = rd_h(b + 108);
    const uint8_t* s = b + 96;
    for (int e = 0; e < 256; e++) {
        const int n = e / 128, j = (e % 128) / 32, l = e % 32;
        const int is = 8 * n + 2 * j + (l >= 16);
        const int lo4 = is < 8 ? (s[is] & 0x0F) : (s[is - 8] >> 4);
        const int hi2 = (s[8 + is % 4] >> (2 * (is / 4))) & 3;
        const int sc = (lo4 | (hi2 << 4)) - 32;
        const int q = (int)((b[32 + 32 * n + l] >> (2 * j)) & 3) - (((b[l] >> (4 * n + j)) & 1) ? 0 : 4);
        y[e] = d * (float)sc * (float)q;
    }
}

/* Q8_K: d f32 @0, qs i8[256] @4, bsums i16[16] @260 (sums of 16 quants each; not used by the values).  y = d * q. */
static void deq_q8_k_block(const uint8_t* b, float* y) {
    float d;
    memcpy(&d, b, 4);
    for (int e = 0; e < 256; e++) y[e] = d * (float)(int8_t)b[4 + e];
}

/* the sixteen values of the non-linear 4-bit formats */
static const int8_t kIq4nl[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

/* IQ4_NL: d f16 @0, qs u8[16] @2.  Low nibbles are elements 0..15, high nibbles 16..31; y = d * table[q]. */
static void deq_iq4_nl_block(const uint8_t* b, float* y) {
    const float d = rd_h(b);
    for (int j = 0; j < 16; j++) {
        y[j] = d * (float)kIq4nl[b[2 + j] & 0x0F];
        y[j + 16] = d * (float)kIq4nl[b[2 + j] >> 4];
    }
}

/* IQ4_XS: d f16 @0, scales_h u16 @2, scales_l u8[4] @4, qs u8[128] @8.  Eight sub-blocks of 32 with a 6-bit
 * scale (low 4 bits in the nibbles of scales_l, high 2 bits in scales_h), offset 32; values as IQ4_NL. */
static void deq_iq4_xs_block(const uint8_t* b, float* y) {
    const float d = rd_h(b);
    const unsigned sh = (unsigned)b[2] | ((unsigned)b[3] << 8);
    for (int ib = 0; ib < 8; ib++) {
        const int ls = ((b[4 + ib / 2] >> (4 * (ib % 2))) & 0x0F) | (int)(((sh >> (2 * ib)) & 3u) << 4);
        const float dl = d * (float)(ls - 32);
        const uint8_t* qs = b + 8 + 16 * ib;
        for (int j = 0; j < 16; j++) {
            y[32 * ib + j] = dl * (float)kIq4nl[qs[j] & 0x0F];
            y[32 * ib + j + 16] = dl * (float)kIq4nl[qs[j] >> 4];
        }
    }
}

/* TQ1_0 (ternary, 1.6875 bits per weight): qs u8[48] @0, qh u8[4] @48, d f16 @52.  A byte packs five trits
 * (four in qh) as a base-3 fraction: byte = ceil(v * 256 / 243), v = sum t_n 3^(4-n); trit n comes back as
 * ((byte * 3^n mod 256) * 3) >> 8.  Elements: trit n of bytes 0..31 at 32 n + m, then trit n of bytes 32..47 at
 * 160 + 16 n + m, then trit n (n < 4) of qh byte j at 240 + 4 n + j.  y = d * (t - 1). */
static void deq_tq1_0_block(const uint8_t* b, float* y) {
    static const uint8_t pow3[5] = {1, 3, 9, 27, 81};
    const float d = rd_h(b + 52);
    for (int n = 0; n < 5; n++)
        for (int m = 0; m < 32; m++) {
            const uint8_t q = (uint8_t)(b[m] * pow3[n]);
            y[32 * n + m] = (float)((int)(((unsigned)q * 3u) >> 8) - 1) * d;
        }
    for (int n = 0; n < 5; n++)
        for (int m = 0; m < 16; m++) {
            const uint8_t q = (uint8_t)(b[32 + m] * pow3[n]);
            y[160 + 16 * n + m] = (float)((int)(((unsigned)q * 3u) >> 8) - 1) * d;
        }
    for (int n = 0; n < 4; n++)
        for (int j = 0; j < 4; j++) {
            const uint8_t q = (uint8_t)(b[48 + j] * pow3[n]);
            y[240 + 4 * n + j] = (float)((int)(((unsigned)q * 3u) >> 8) - 1) * d;
        }
}

/* TQ2_0 (ternary, 2.0625 bits per weight): qs u8[64] @0, d f16 @64.  Element 128 g + 32 l + m is bits 2l..2l+1
 * of byte 32 g + m; y = d * (q - 1). */
static void deq_tq2_0_block(const uint8_t* b, float* y) {
    const float d = rd_h(b + 64);
    for (int g = 0; g < 2; g++)
        for (int l = 0; l < 4; l++)
            for (int m = 0; m < 32; m++) y[128 * g + 32 * l + m] = (float)((int)((b[32 * g + m] >> (2 * l)) & 3) - 1) * d;
}

static int is_block_type(int type) {
    return type == T_Q8_0 || type == T_Q4_K || type == T_Q6_K || type == T_Q4_0 || type == T_Q4_1 || type == T_Q5_0 ||
           type == T_Q5_1 || type == T_Q2_K || type == T_Q5_K || type == T_F16 || type == T_BF16 || type == T_F32 ||
           type == T_Q3_K || type == T_Q8_K || type == T_IQ4_NL || type == T_IQ4_XS || type == T_TQ1_0 || type == T_TQ2_0;
}

static void deq_block(int type, const uint8_t* b, float* y) {
    uint16_t h;
    switch (type) {
        case T_Q8_0: deq_q8_0_block(b, y); break;
        case T_Q4_K: deq_q4_k_block(b, y); break;
        case T_Q6_K: deq_q6_k_block(b, y); break;
        case T_Q4_0: deq_q4_0_block(b, y); break;
        case T_Q4_1: deq_q4_1_block(b, y); break;
        case T_Q5_0: deq_q5_0_block(b, y); break;
        case T_Q5_1: deq_q5_1_block(b, y); break;
        case T_Q2_K: deq_q2_k_block(b, y); break;
        case T_Q5_K: deq_q5_k_block(b, y); break;
        case T_Q3_K: deq_q3_k_block(b, y); break;
        case T_Q8_K: deq_q8_k_block(b, y); break;
        case T_IQ4_NL: deq_iq4_nl_block(b, y); break;
        case T_IQ4_XS: deq_iq4_xs_block(b, y); break;
        case T_TQ1_0: deq_tq1_0_block(b, y); break;
        case T_TQ2_0: deq_tq2_0_block(b, y); break;
        case T_F16: memcpy(&h, b, 2); y[0] = orc_h2f(h); break;
        case T_BF16: memcpy(&h, b, 2); y[0] = orc_bf2f(h); break;
        default: memcpy(y, b, 4); break; /* F32 */
    }
}

/* n_elems consecutive elements (a block multiple) of `type` -> fp32. */
int orc_dequant(int type, const uint8_t* w, int64_t n_elems, float* out) {
    int be, bb;
    if (!is_block_type(type)) return ORC_ERR_TYPE;
    orc_type_sizes(type, &be, &bb);
    if (n_elems < 0 || n_elems % be != 0) return ORC_ERR_SHAPE;
    const int64_t nb = n_elems / be;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < nb; i++) deq_block(type, w + i * bb, out + i * be);
    return ORC_OK;
}

/* --------------------------------------------------------- dense reference */

/* DoublesTensor.kt:255-264: y[j] = sum_i x[i] * B[i*N + j], i outer, fp64. */
void orc_dense_vecmat(const double* x, const double* B, int K, int N, double* y) {
    for (int j = 0; j < N; j++) y[j] = 0.0;
    for (int i = 0; i < K; i++)
        for (int j = 0; j < N; j++) y[j] += x[i] * B[(int64_t)i * N + j];
}

/* DoublesTensor.kt:267-279: naive i-j-k, fp64. */
void orc_dense_matmul(const double* A, const double* B, int M, int K, int N, double* C) {
    for (int i = 0; i < M; i++)
        for (int j = 0; j < N; j++) {
            double s = 0.0;
            for (int k = 0; k < K; k++) s += A[(int64_t)i * K + k] * B[(int64_t)k * N + j];
            C[(int64_t)i * N + j] = s;
        }
}

/* ------------------------------------------------------- quantized matvec */

/* y[n] = sum_k deq(W)[n,k] * x[k]; W is N rows of K/blk blocks ([out,in] as in Linear.kt:26-28).
 * Accumulates in fp64 (the reference's arithmetic type), rounds once to fp32. */
int orc_matvec_q(int type, const uint8_t* w, int N, int K, const float* x, float* y) {
    int64_t rb = orc_row_bytes(type, K);
    if (rb < 0) return (int)rb;
    if (!is_block_type(type)) return ORC_ERR_TYPE;
    int be, bb;
    orc_type_sizes(type, &be, &bb);
    const int nb = K / be;
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; n++) {
        float tmp[256];
        double acc = 0.0;
        const uint8_t* row = w + (int64_t)n * rb;
        for (int b = 0; b < nb; b++) {
            deq_block(type, row + (int64_t)b * bb, tmp);
            const float* xb = x + (int64_t)b * be;
            for (int i = 0; i < be; i++) acc += (double)tmp[i] * (double)xb[i];
        }
        y[n] = (float)acc;
    }
    return ORC_OK;
}

/* The reference's own algorithm for a Linear with such a weight today: dequantize to fp64,
 * materialise the transpose (DoublesTensor.kt:362-387, called per forward by Linear.kt:48), then the
 * i-outer vec x mat loop (DoublesTensor.kt:255-264).  Single thread, like the reference. */
int orc_matvec_q_reference_algorithm(int type, const uint8_t* w, int N, int K, const float* x, float* y) {
    int64_t rb = orc_row_bytes(type, K);
    if (rb < 0) return (int)rb;
    float* wf = (float*)malloc((size_t)N * K * sizeof(float));
    double* wd = (double*)malloc((size_t)N * K * sizeof(double));
    double* wt = (double*)malloc((size_t)N * K * sizeof(double));
    double* xd = (double*)malloc((size_t)K * sizeof(double));
    double* yd = (double*)malloc((size_t)N * sizeof(double));
    if (!wf || !wd || !wt || !xd || !yd) { free(wf); free(wd); free(wt); free(xd); free(yd); return -4; }
    int be, bb;
    orc_type_sizes(type, &be, &bb);
    for (int64_t i = 0; i < (int64_t)N * K / be; i++) deq_block(type, w + i * bb, wf + i * be);
    for (int64_t i = 0; i < (int64_t)N * K; i++) wd[i] = wf[i];
    for (int i = 0; i < N; i++)
        for (int j = 0; j < K; j++) wt[(int64_t)j * N + i] = wd[(int64_t)i * K + j];
    for (int k = 0; k < K; k++) xd[k] = x[k];
    orc_dense_vecmat(xd, wt, K, N, yd);
    for (int n = 0; n < N; n++) y[n] = (float)yd[n];
    free(wf); free(wd); free(wt); free(xd); free(yd);
    return ORC_OK;
}

/* C[m,n] = sum_k A[m,k] * deq(W)[n,k]; A bf16 [M,K], C fp32 [M,N]; fp64 accumulate. */
int orc_gemm_q(int type, const uint8_t* w, int N, int K, const uint16_t* a_bf16, int M, float* c) {
    int64_t rb = orc_row_bytes(type, K);
    if (rb < 0) return (int)rb;
    if (!is_block_type(type)) return ORC_ERR_TYPE;
    int be, bb;
    orc_type_sizes(type, &be, &bb);
    float* af = (float*)malloc((size_t)M * K * sizeof(float));
    if (!af) return -4;
    for (int64_t i = 0; i < (int64_t)M * K; i++) af[i] = orc_bf2f(a_bf16[i]);
#pragma omp parallel
    {
        float* wrow = (float*)malloc((size_t)K * sizeof(float));
#pragma omp for schedule(static)
        for (int n = 0; n < N; n++) {
            const uint8_t* row = w + (int64_t)n * rb;
            for (int b = 0; b < K / be; b++) deq_block(type, row + (int64_t)b * bb, wrow + (int64_t)b * be);
            for (int m = 0; m < M; m++) {
                const float* ar = af + (int64_t)m * K;
                double acc = 0.0;
                for (int k = 0; k < K; k++) acc += (double)ar[k] * (double)wrow[k];
                c[(int64_t)m * N + n] = (float)acc;
            }
        }
        free(wrow);
    }
    free(af);
    return ORC_OK;
}

/* ------------------------------------------------------- decode attention */

/* One (sequence, head): o = softmax(q . K^T * scale) . V over n_ctx tokens.
 * k, v: fp16 bits, token-major [n_ctx][stride] with this head's `dim` values at k + t*stride.
 * Max-subtracted textbook softmax in fp64. */
void orc_attn_head(const float* q, const uint16_t* k, const uint16_t* v, int n_ctx, int dim, int64_t stride,
                   double scale, float* out) {
    double* s = (double*)malloc((size_t)n_ctx * sizeof(double));
    double mx = -INFINITY;
    for (int t = 0; t < n_ctx; t++) {
        double acc = 0.0;
        for (int d = 0; d < dim; d++) acc += (double)q[d] * (double)orc_h2f(k[t * stride + d]);
        s[t] = acc * scale;
        if (s[t] > mx) mx = s[t];
    }
    double den = 0.0;
    for (int t = 0; t < n_ctx; t++) { s[t] = exp(s[t] - mx); den += s[t]; }
    for (int d = 0; d < dim; d++) {
        double acc = 0.0;
        for (int t = 0; t < n_ctx; t++) acc += s[t] * (double)orc_h2f(v[t * stride + d]);
        out[d] = (float)(acc / den);
    }
    free(s);
}

/* Batched: q/out fp32 [n_seq][n_head][dim]; k,v flat fp16 [n_seq][max_tokens][n_head][dim];
 * n_ctx[s] tokens attended for sequence s. */
void orc_attn_decode(const float* q, const uint16_t* k, const uint16_t* v, const int32_t* n_ctx, int n_seq,
                     int n_head, int dim, int max_tokens, double scale, float* out) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int s = 0; s < n_seq; s++)
        for (int h = 0; h < n_head; h++) {
            const int64_t base = ((int64_t)s * max_tokens * n_head + h) * dim;
            orc_attn_head(q + ((int64_t)s * n_head + h) * dim, k + base, v + base, n_ctx[s], dim,
                          (int64_t)n_head * dim, scale, out + ((int64_t)s * n_head + h) * dim);
        }
}

/* ------------------------------------------------------------ decoder glue */

/* y = x / sqrt(mean(x^2) + eps) * w, fp64 inside. */
void orc_rmsnorm(const float* x, const float* w, int n, double eps, float* y) {
    double ss = 0.0;
    for (int i = 0; i < n; i++) ss += (double)x[i] * (double)x[i];
    double r = 1.0 / sqrt(ss / n + eps);
    for (int i = 0; i < n; i++) y[i] = (float)((double)x[i] * r * (double)w[i]);
}

/* Rotary embedding, interleaved pairs (2i, 2i+1) within each head, angle = pos * base^(-2i/dim). */
void orc_rope(float* x, int n_head, int dim, int pos, double base) {
    for (int h = 0; h < n_head; h++)
        for (int i = 0; i < dim / 2; i++) {
            double theta = (double)pos * pow(base, -2.0 * i / dim);
            double c = cos(theta), s = sin(theta);
            float* p = x + (int64_t)h * dim + 2 * i;
            double a = p[0], b = p[1];
            p[0] = (float)(a * c - b * s);
            p[1] = (float)(a * s + b * c);
        }
}

/* out = silu(gate) * up. */
void orc_swiglu(const float* gate, const float* up, int n, float* out) {
    for (int i = 0; i < n; i++) {
        double g = gate[i];
        out[i] = (float)(g / (1.0 + exp(-g)) * (double)up[i]);
    }
}

/* First index of the maximum (the reference's inline argmax keeps the first maximum too:
 * samples/mnist-mlp-cli/src/jvmMain/kotlin/.../Main.kt:269-278 uses a strict '>' scan). */
int orc_argmax(const float* x, int n) {
    int best = 0;
    for (int i = 1; i < n; i++)
        if (x[i] > x[best]) best = i;
    return best;
}

int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void orc_set_num_threads(int n) {
#ifdef _OPENMP
    omp_set_num_threads(n);
#else
    (void)n;
#endif
}
