// The further ggml formats of the reference's size table (gguf/.../Constants.kt:58-90) that the library
// computes with: Q4_0, Q4_1, Q5_0, Q5_1, Q2_K, Q3_K, Q5_K, Q8_K, IQ4_NL, IQ4_XS, TQ1_0, TQ2_0 and the dense
// F32 / F16 / BF16.  One decode function per
// format -- four consecutive elements of a block at a time, every value the exact real of its formula rounded
// once (explicitly rounded intrinsics, so no contraction can change a bit) -- serves a dequantization kernel
// (one thread per four outputs, 16-byte stores) and a batch-1 matvec (one wavefront per row, the lane's four
// weights against one aligned float4 of x, DPP reduction; for blocks of a multiple of four bytes the row passes
// through LDS first).  These are plain streaming kernels: Q5_K, Q4_0, Q4_1, Q5_0, Q5_1 and IQ4_NL reach them only when a
// row or pointer is off the 16-byte grid -- otherwise their matvec runs on the lane map of the Q4_K kernel
// (matvec.hip), like the hand-tuned Q4_K, Q8_0 and Q6_K.
#include "common.h"

namespace {

typedef uint32_t u32_a2 __attribute__((aligned(2)));

__device__ __forceinline__ uint32_t ld32(const uint8_t* p) { return *reinterpret_cast<const u32_a2*>(p); }
__device__ __forceinline__ float ldh(const uint8_t* p) { return h2f_bits(*reinterpret_cast<const uint16_t*>(p)); }

template <int T>
struct Fmt;

// Q4_0, 18 B: f16 d @0, qs[16] @2.  Low nibbles are elements 0..15, high nibbles 16..31; y = d * (q - 8).
template <>
struct Fmt<SKN_TYPE_Q4_0> {
    static constexpr int kElems = 32, kBytes = 18;
    static __device__ __forceinline__ float4 decode4(const uint8_t* b, int g) {
        const float d = ldh(b);
        uint32_t q = ld32(b + 2 + 4 * (g & 3));
        if (g >= 4) q >>= 4;
        float4 y;
        y.x = __fmul_rn(d, (float)((int)(q & 0xF) - 8));
        y.y = __fmul_rn(d, (float)((int)((q >> 8) & 0xF) - 8));
        y.z = __fmul_rn(d, (float)((int)((q >> 16) & 0xF) - 8));
        y.w = __fmul_rn(d, (float)((int)((q >> 24) & 0xF) - 8));
        return y;
    }
};

// Q4_1, 20 B: f16 d @0, f16 m @2, qs[16] @4.  y = d * q + m.
template <>
struct Fmt<SKN_TYPE_Q4_1> {
    static constexpr int kElems = 32, kBytes = 20;
    static __device__ __forceinline__ float4 decode4(const uint8_t* b, int g) {
        const float d = ldh(b), m = ldh(b + 2);
        uint32_t q = ld32(b + 4 + 4 * (g & 3));
        if (g >= 4) q >>= 4;
        float4 y;
        y.x = __fadd_rn(__fmul_rn(d, (float)(q & 0xF)), m);
        y.y = __fadd_rn(__fmul_rn(d, (float)((q >> 8) & 0xF)), m);
        y.z = __fadd_rn(__fmul_rn(d, (float)((q >> 16) & 0xF)), m);
        y.w = __fadd_rn(__fmul_rn(d, (float)((q >> 24) & 0xF)), m);
        return y;
    }
};

// five-bit values of elements 4g .. 4g+3: nibbles of qs[4 (g % 4) ..] (low for g < 4) with bit (element) of qh
__device__ __forceinline__ void q5_quad(uint32_t qs4, uint32_t qh, int g, int (&v)[4]) {
    if (g >= 4) qs4 >>= 4;
    const uint32_t hb = qh >> (4 * g);
#pragma unroll
    for (int i = 0; i < 4; i++) v[i] = (int)(((qs4 >> (8 * i)) & 0xF) | (((hb >> i) & 1u) << 4));
}

// Q5_0, 22 B: f16 d @0, u32 qh @2 (bit j = fifth bit of element j), qs[16] @6.  y = d * (q - 16).
template <>
struct Fmt<SKN_TYPE_Q5_0> {
    static constexpr int kElems = 32, kBytes = 22;
    static __device__ __forceinline__ float4 decode4(const uint8_t* b, int g) {
        const float d = ldh(b);
        int v[4];
        q5_quad(ld32(b + 6 + 4 * (g & 3)), ld32(b + 2), g, v);
        return make_float4(__fmul_rn(d, (float)(v[0] - 16)), __fmul_rn(d, (float)(v[1] - 16)),
                           __fmul_rn(d, (float)(v[2] - 16)), __fmul_rn(d, (float)(v[3] - 16)));
    }
};

// Q5_1, 24 B: f16 d @0, f16 m @2, u32 qh @4, qs[16] @8.  y = d * q + m.
template <>
struct Fmt<SKN_TYPE_Q5_1> {
    static constexpr int kElems = 32, kBytes = 24;
    static __device__ __forceinline__ float4 decode4(const uint8_t* b, int g) {
        const float d = ldh(b), m = ldh(b + 2);
        int v[4];
        q5_quad(ld32(b + 8 + 4 * (g & 3)), ld32(b + 4), g, v);
        return make_float4(__fadd_rn(__fmul_rn(d, (float)v[0]), m), __fadd_rn(__fmul_rn(d, (float)v[1]), m),
                           __fadd_rn(__fmul_rn(d, (float)v[2]), m), __fadd_rn(__fmul_rn(d, (float)v[3]), m));
    }
};

// Q2_K, 84 B: scales[16] @0 (low nibble scale, high nibble min), qs[64] @16, f16 d @80, f16 dmin @82.
// Element e: half n = e / 128, bit pair j = (e % 128) / 32, l = e % 32: qs[32n + l] >> 2j, scale 8n + 2j + (l >= 16).
template <>
struct Fmt<SKN_TYPE_Q2_K> {
    static constexpr int kElems = 256, kBytes = 84;
    static __device__ __forceinline__ float4 decode4(const uint8_t* b, int g) {
        const int e = 4 * g, n = e >> 7, j = (e & 127) >> 5, l = e & 31;
        const uint32_t s = b[8 * n + 2 * j + (l >> 4)];
        const float dl = __fmul_rn(ldh(b + 80), (float)(s & 0xF));
        const float ml = __fmul_rn(ldh(b + 82), (float)(s >> 4));
        const uint32_t q = ld32(b + 16 + 32 * n + l) >> (2 * j);
        float4 y;
        y.x = __fsub_rn(__fmul_rn(dl, (float)(q & 3)), ml);
        y.y = __fsub_rn(__fmul_rn(dl, (float)((q >> 8) & 3)), ml);
        y.z = __fsub_rn(__fmul_rn(dl, (float)((q >> 16) & 3)), ml);
        y.w = __fsub_rn(__fmul_rn(dl, (float)((q >> 24) & 3)), ml);
        return y;
    }
};

// Q5_K, 176 B: f16 d @0, f16 dmin @2, scales[12] @4 (the Q4_K packing), qh[32] @16, qs[128] @48.
// Element e: chunk c = e / 64, r = e % 64, sub-block 2c + (r >= 32); nibble of qs[32c + r % 32], fifth bit =
// bit (sub-block) of qh[r % 32].
template <>
struct Fmt<SKN_TYPE_Q5_K> {
    static constexpr int kElems = 256, kBytes = 176;
    static __device__ __forceinline__ float4 decode4(const uint8_t* b, int g) {
        const int e = 4 * g, c = e >> 6, r = e & 63, up = r >> 5, j = 2 * c + up, l = r & 31;
        const uint8_t* s = b + 4;
        int sc, m;
        if (j < 4) {
            sc = s[j] & 63;
            m = s[j + 4] & 63;
        } else {
            sc = (s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4);
            m = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
        }
        const float d1 = __fmul_rn(ldh(b), (float)sc), m1 = __fmul_rn(ldh(b + 2), (float)m);
        uint32_t q = ld32(b + 48 + 32 * c + l);
        if (up) q >>= 4;
        const uint32_t hb = ld32(b + 16 + l) >> j;
        float4 y;
        y.x = __fsub_rn(__fmul_rn(d1, (float)((q & 0xF) | ((hb & 1) << 4))), m1);
        y.y = __fsub_rn(__fmul_rn(d1, (float)(((q >> 8) & 0xF) | (((hb >> 8) & 1) << 4))), m1);
        y.z = __fsub_rn(__fmul_rn(d1, (float)(((q >> 16) & 0xF) | (((hb >> 16) & 1) << 4))), m1);
        y.w = __fsub_rn(__fmul_rn(d1, (float)(((q >> 24) & 0xF) | (((hb >> 24) & 1) << 4))), m1);
        return y;
    }
};

// Q3_K, 110 B: hmask[32] @0, qs[64] @32, scales[12] @96, f16 d @108.  Sixteen 6-bit scales stored with an offset
// of 32: low nibbles of bytes 0..7 for scales 0..7, high nibbles for 8..15, two more bits each from bytes 8..11.
// Element e: half n = e / 128, bit pair j = (e % 128) / 32, l = e % 32: two bits of qs[32n + l] at 2j, minus 4
// unless bit 4n + j of hmask[l] is set; scale 8n + 2j + (l >= 16).
template <>
struct Fmt<SKN_TYPE_Q3_K> {
    static constexpr int kElems = 256, kBytes = 110;
    static __device__ __forceinline__ float4 decode4(const uint8_t* b, int g) {
        const int e = 4 * g, n = e >> 7, j = (e & 127) >> 5, l = e & 31;
        const int is = 8 * n + 2 * j + (l >> 4);
        const uint8_t* s = b + 96;
        const int lo4 = is < 8 ? (s[is] & 0x0F) : (s[is - 8] >> 4);
        const int hi2 = (s[8 + (is & 3)] >> (2 * (is >> 2))) & 3;
        const float dl = __fmul_rn(ldh(b + 108), (float)((lo4 | (hi2 << 4)) - 32));
        const uint32_t q = ld32(b + 32 + 32 * n + l) >> (2 * j);
        const uint32_t hb = ld32(b + l) >> (4 * n + j);
        float4 y;
        y.x = __fmul_rn(dl, (float)((int)(q & 3) - ((hb & 1) ? 0 : 4)));
        y.y = __fmul_rn(dl, (float)((int)((q >> 8) & 3) - (((hb >> 8) & 1) ? 0 : 4)));
        y.z = __fmul_rn(dl, (float)((int)((q >> 16) & 3) - (((hb >> 16) & 1) ? 0 : 4)));
        y.w = __fmul_rn(dl, (float)((int)((q >> 24) & 3) - (((hb >> 24) & 1) ? 0 : 4)));
        return y;
    }
};

// Q8_K, 292 B: f32 d @0, int8 qs[256] @4, int16 block sums @260 (not part of the values).  y = d * q.
template <>
struct Fmt<SKN_TYPE_Q8_K> {
    static constexpr int kElems = 256, kBytes = 292;
    static __device__ __forceinline__ float4 decode4(const uint8_t* b, int g) {
        const float d = __uint_as_float(ld32(b));
        const uint32_t q = ld32(b + 4 + 4 * g);
        return make_float4(__fmul_rn(d, (float)(int8_t)(q & 0xFF)), __fmul_rn(d, (float)(int8_t)((q >> 8) & 0xFF)),
                           __fmul_rn(d, (float)(int8_t)((q >> 16) & 0xFF)), __fmul_rn(d, (float)(int8_t)(q >> 24)));
    }
};

// the sixteen values of the non-linear 4-bit formats, packed four to a word (index = nibble)
__device__ __forceinline__ float iq4_value(uint32_t nibble) {
    const uint32_t tab[4] = {0xBFAD9881u, 0xF6EADDCFu, 0x26190D01u, 0x71594535u};  // -127,-104,-83,-65 | -49,-35,-22,-10 | 1,13,25,38 | 53,69,89,113
    const uint32_t w = nibble < 8 ? (nibble < 4 ? tab[0] : tab[1]) : (nibble < 12 ? tab[2] : tab[3]);
    return (float)(int8_t)((w >> (8 * (nibble & 3))) & 0xFF);
}

// IQ4_NL, 18 B: f16 d @0, qs[16] @2.  Low nibbles are elements 0..15, high nibbles 16..31; y = d * table[q].
template <>
struct Fmt<SKN_TYPE_IQ4_NL> {
    static constexpr int kElems = 32, kBytes = 18;
    static __device__ __forceinline__ float4 decode4(const uint8_t* b, int g) {
        const float d = ldh(b);
        uint32_t q = ld32(b + 2 + 4 * (g & 3));
        if (g >= 4) q >>= 4;
        return make_float4(__fmul_rn(d, iq4_value(q & 0xF)), __fmul_rn(d, iq4_value((q >> 8) & 0xF)),
                           __fmul_rn(d, iq4_value((q >> 16) & 0xF)), __fmul_rn(d, iq4_value((q >> 24) & 0xF)));
    }
};

// IQ4_XS, 136 B: f16 d @0, u16 scales_h @2, scales_l[4] @4, qs[128] @8.  Eight sub-blocks of 32 with a 6-bit scale
// (low 4 bits in the nibbles of scales_l, high 2 bits in scales_h) stored with an offset of 32; values as IQ4_NL.
template <>
struct Fmt<SKN_TYPE_IQ4_XS> {
    static constexpr int kElems = 256, kBytes = 136;
    static __device__ __forceinline__ float4 decode4(const uint8_t* b, int g) {
        const int ib = g >> 3, gg = g & 7;
        const uint32_t sh = *reinterpret_cast<const uint16_t*>(b + 2);
        const int ls = (int)(((b[4 + (ib >> 1)] >> (4 * (ib & 1))) & 0x0F) | (((sh >> (2 * ib)) & 3u) << 4));
        const float dl = __fmul_rn(ldh(b), (float)(ls - 32));
        uint32_t q = ld32(b + 8 + 16 * ib + 4 * (gg & 3));
        if (gg >= 4) q >>= 4;
        return make_float4(__fmul_rn(dl, iq4_value(q & 0xF)), __fmul_rn(dl, iq4_value((q >> 8) & 0xF)),
                           __fmul_rn(dl, iq4_value((q >> 16) & 0xF)), __fmul_rn(dl, iq4_value((q >> 24) & 0xF)));
    }
};

// TQ1_0 (ternary), 54 B: qs[48] @0, qh[4] @48, f16 d @52.  A byte packs five trits (four in qh) as a base-3
// fraction, byte = ceil(v * 256 / 243) with v = sum t_n 3^(4-n); trit n is ((byte * 3^n mod 256) * 3) >> 8.
// Elements: trit n of bytes 0..31 at 32 n + m; trit n of bytes 32..47 at 160 + 16 n + m; trit n (< 4) of qh byte
// j at 240 + 4 n + j.  y = d * (t - 1).
template <>
struct Fmt<SKN_TYPE_TQ1_0> {
    static constexpr int kElems = 256, kBytes = 54;
    static __device__ __forceinline__ float4 decode4(const uint8_t* b, int g) {
        const int e = 4 * g;
        int n, off;
        if (e < 160) n = e >> 5, off = e & 31;
        else if (e < 240) n = (e - 160) >> 4, off = 32 + ((e - 160) & 15);
        else n = (e - 240) >> 2, off = 48;
        const uint32_t p3 = n == 0 ? 1u : n == 1 ? 3u : n == 2 ? 9u : n == 3 ? 27u : 81u;
        const uint32_t q = ld32(b + off);
        const float d = ldh(b + 52);
        float y[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t t = ((((q >> (8 * i)) & 0xFFu) * p3 & 0xFFu) * 3u) >> 8;
            y[i] = __fmul_rn((float)((int)t - 1), d);
        }
        return make_float4(y[0], y[1], y[2], y[3]);
    }
};

// TQ2_0 (ternary), 66 B: qs[64] @0, f16 d @64.  Element 128 g + 32 l + m is bits 2l..2l+1 of byte 32 g + m;
// y = d * (q - 1).
template <>
struct Fmt<SKN_TYPE_TQ2_0> {
    static constexpr int kElems = 256, kBytes = 66;
    static __device__ __forceinline__ float4 decode4(const uint8_t* b, int g) {
        const int e = 4 * g, l = (e >> 5) & 3;
        const uint32_t q = ld32(b + 32 * (e >> 7) + (e & 31)) >> (2 * l);
        const float d = ldh(b + 64);
        return make_float4(__fmul_rn((float)((int)(q & 3) - 1), d), __fmul_rn((float)((int)((q >> 8) & 3) - 1), d),
                           __fmul_rn((float)((int)((q >> 16) & 3) - 1), d), __fmul_rn((float)((int)((q >> 24) & 3) - 1), d));
    }
};

// The three formats with tuned kernels of their own, decoded here as well for the GEMM's weight pass (same
// arithmetic as the dequantization kernels: every value the exact real of its formula rounded once).
// Q8_0, 34 B: f16 d @0, int8 qs[32] @2.
template <>
struct Fmt<SKN_TYPE_Q8_0> {
    static constexpr int kElems = 32, kBytes = 34;
    static __device__ __forceinline__ float4 decode4(const uint8_t* b, int g) {
        const float d = ldh(b);
        const uint32_t q = ld32(b + 2 + 4 * g);
        return make_float4(__fmul_rn(d, (float)(int8_t)(q & 0xFF)), __fmul_rn(d, (float)(int8_t)((q >> 8) & 0xFF)),
                           __fmul_rn(d, (float)(int8_t)((q >> 16) & 0xFF)), __fmul_rn(d, (float)(int8_t)(q >> 24)));
    }
};

// Q4_K, 144 B: f16 d @0, f16 dmin @2, 12 packed 6-bit scale / min bytes @4, 128 nibble bytes @16.
template <>
struct Fmt<SKN_TYPE_Q4_K> {
    static constexpr int kElems = 256, kBytes = 144;
    static __device__ __forceinline__ float4 decode4(const uint8_t* b, int g) {
        const int e = 4 * g, c = e >> 6, r = e & 63, j = 2 * c + (r >= 32);
        const float d = ldh(b), dmin = ldh(b + 2);
        const uint8_t* s = b + 4;
        int sc, m;
        if (j < 4) {
            sc = s[j] & 63;
            m = s[j + 4] & 63;
        } else {
            sc = (s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4);
            m = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
        }
        uint32_t q = ld32(b + 16 + 32 * c + (r & 31));
        if (r >= 32) q >>= 4;
        const float d1 = __fmul_rn(d, (float)sc), m1 = __fmul_rn(dmin, (float)m);
        return make_float4(__fsub_rn(__fmul_rn(d1, (float)(q & 0xF)), m1), __fsub_rn(__fmul_rn(d1, (float)((q >> 8) & 0xF)), m1),
                           __fsub_rn(__fmul_rn(d1, (float)((q >> 16) & 0xF)), m1),
                           __fsub_rn(__fmul_rn(d1, (float)((q >> 24) & 0xF)), m1));
    }
};

// Q6_K, 210 B: ql[128] @0 (low nibbles), qh[64] @128 (high bit pairs), int8 scales[16] @192, f16 d @208.
template <>
struct Fmt<SKN_TYPE_Q6_K> {
    static constexpr int kElems = 256, kBytes = 210;
    static __device__ __forceinline__ float4 decode4(const uint8_t* b, int g) {
        const int e = 4 * g, n = e >> 7, r = e & 127, quarter = r >> 5, l = r & 31;
        uint32_t lo = ld32(b + 64 * n + l + 32 * (quarter & 1));
        if (quarter >= 2) lo >>= 4;
        const uint32_t hi = ld32(b + 128 + 32 * n + l) >> (2 * quarter);
        const float ds = __fmul_rn(ldh(b + 208), (float)(int8_t)b[192 + 8 * n + 2 * quarter + (l >> 4)]);
        return make_float4(__fmul_rn(ds, (float)((int)((lo & 0xF) | ((hi & 3) << 4)) - 32)),
                           __fmul_rn(ds, (float)((int)(((lo >> 8) & 0xF) | (((hi >> 8) & 3) << 4)) - 32)),
                           __fmul_rn(ds, (float)((int)(((lo >> 16) & 0xF) | (((hi >> 16) & 3) << 4)) - 32)),
                           __fmul_rn(ds, (float)((int)(((lo >> 24) & 0xF) | (((hi >> 24) & 3) << 4)) - 32)));
    }
};

// Dense rows, read a scalar at a time where a caller needs it and four at a time otherwise.
template <int T>
__device__ __forceinline__ float dense_at(const uint8_t* w, int64_t i) {
    if (T == SKN_TYPE_F32) return reinterpret_cast<const float*>(w)[i];
    const uint32_t bits = reinterpret_cast<const uint16_t*>(w)[i];
    return T == SKN_TYPE_F16 ? h2f_bits(bits) : __uint_as_float(bits << 16);
}

template <int T>
__global__ __launch_bounds__(256) void dequant_blocks_kernel(const uint8_t* __restrict__ w, float* __restrict__ out,
                                                             int64_t n_quads) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_quads) return;
    constexpr int QB = Fmt<T>::kElems / 4;  // quads per block
    reinterpret_cast<float4*>(out)[t] = Fmt<T>::decode4(w + (t / QB) * Fmt<T>::kBytes, (int)(t % QB));
}

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));

// four consecutive elements 4q .. 4q + 3 of a weight row
template <int T>
__device__ __forceinline__ float4 row_quad(const uint8_t* row, int q) {
    if constexpr (T == SKN_TYPE_F32 || T == SKN_TYPE_F16 || T == SKN_TYPE_BF16) {
        return make_float4(dense_at<T>(row, 4 * q), dense_at<T>(row, 4 * q + 1), dense_at<T>(row, 4 * q + 2),
                           dense_at<T>(row, 4 * q + 3));
    } else {
        constexpr int QB = Fmt<T>::kElems / 4;
        return Fmt<T>::decode4(row + (size_t)(q / QB) * Fmt<T>::kBytes, q % QB);
    }
}

template <int T>
__host__ __device__ constexpr size_t row_bytes_of(int k) {
    if constexpr (T == SKN_TYPE_F32) return (size_t)k * 4;
    else if constexpr (T == SKN_TYPE_F16 || T == SKN_TYPE_BF16) return (size_t)k * 2;
    else return (size_t)(k / Fmt<T>::kElems) * Fmt<T>::kBytes;
}

// The GEMM's weight pass: W [n, k] of any format -> an fp16 pair (hi = f16(w), lo = f16((w - hi) * 2^11)) in the
// order in which the matrix-core kernel consumes it.  For a block of 32 weight rows and a k-step t (sixteen
// elements) the 64 x 16 bytes that the 64 lanes hand to one matrix instruction are contiguous, hi operand then lo
// operand: piece ((cb * steps + t) * 2 + hl) * 64 + 32 h + r, where lane (h, r) holds row r and -- with
// dw = 4 h + t % 4 inside the 64-element chunk t / 4 -- the elements 4 dw + {0, 2}, 32 + 4 dw + {0, 2},
// 4 dw + {1, 3}, 32 + 4 dw + {1, 3}: the order of the activation fragments.  lo is kept times 2^11 so that it is
// a normal fp16 number wherever hi is one (the kernel keeps its products in accumulators of their own).
// One thread per (row, chunk, dw): eight neighbouring threads read 64 consecutive elements of a row.  The
// pieces of the workgroup's 32 rows x kFragChunks chunks -- one contiguous 8 KiB run of the output per chunk -- are
// collected in LDS and written out in order, 1 KiB per wavefront store.  Rows beyond n repeat row n - 1 (their
// products are never stored).
constexpr int kFragChunks = 4;  // chunks per workgroup
template <int T>
__global__ __launch_bounds__(256) void weights_hilo_frag_kernel(const uint8_t* __restrict__ w, half8_t* __restrict__ bfrag,
                                                                int n, int k) {
    __shared__ half8_t stage[kFragChunks * 512];
    const int r = threadIdx.x >> 3, dw = threadIdx.x & 7;
    const int cb = blockIdx.y, steps = k >> 4, nch = k >> 6;
    const uint8_t* row = w + (size_t)min(cb * 32 + r, n - 1) * row_bytes_of<T>(k);
    const int h = dw >> 2, s = dw & 3;
    const int c0 = blockIdx.x * kFragChunks, chunks = min(kFragChunks, nch - c0);
#pragma unroll
    for (int x = 0; x < kFragChunks; x++) {
        if (x >= chunks) break;
        const int c = c0 + x;
        const float4 l = row_quad<T>(row, 16 * c + dw), u = row_quad<T>(row, 16 * c + dw + 8);
        const float v[8] = {l.x, l.z, u.x, u.z, l.y, l.w, u.y, u.w};
        half8_t vh, vl;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            float f = v[i];
            asm("" : "+v"(f));  // (keeps the two conversions of a fused product apart, see skn_split_hilo)
            const _Float16 a = (_Float16)f;
            vh[i] = a;
            vl[i] = (_Float16)((f - (float)a) * 2048.0f);
        }
        half8_t* dst = stage + x * 512 + s * 128 + 32 * h + r;
        dst[0] = vh;
        dst[64] = vl;
    }
    __syncthreads();
    half8_t* out = bfrag + ((size_t)cb * steps + 4 * c0) * 128;
    for (int i = threadIdx.x; i < chunks * 512; i += 256) out[i] = stage[i];
}

template <int T>
__global__ __launch_bounds__(256) void convert_dense_kernel(const uint8_t* __restrict__ w, float* __restrict__ out,
                                                            int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = dense_at<T>(w, i);
}

// one wavefront per row, four rows per workgroup; lane l takes quads l, l + 64, ...
template <int T>
__global__ __launch_bounds__(256) void matvec_blocks_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                            float* __restrict__ y, int n_rows, int k) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n_rows) return;
    constexpr int QB = Fmt<T>::kElems / 4;
    const uint8_t* rowp = w + (size_t)row * (k / Fmt<T>::kElems) * Fmt<T>::kBytes;
    float acc = 0.f;
    const int nq = k >> 2;
    int q = lane;
    // four quads per lane and turn: their loads are issued together, the row is read with four requests in flight
    for (; q + 192 < nq; q += 256) {
        float4 wv[4], xv[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int qq = q + 64 * u;
            wv[u] = Fmt<T>::decode4(rowp + (size_t)(qq / QB) * Fmt<T>::kBytes, qq % QB);
            xv[u] = reinterpret_cast<const float4*>(x)[qq];
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            acc = fmaf(wv[u].x, xv[u].x, acc);
            acc = fmaf(wv[u].y, xv[u].y, acc);
            acc = fmaf(wv[u].z, xv[u].z, acc);
            acc = fmaf(wv[u].w, xv[u].w, acc);
        }
    }
    for (; q < nq; q += 64) {
        const float4 wv = Fmt<T>::decode4(rowp + (size_t)(q / QB) * Fmt<T>::kBytes, q % QB);
        const float4 xv = reinterpret_cast<const float4*>(x)[q];
        acc = fmaf(wv.x, xv.x, acc);
        acc = fmaf(wv.y, xv.y, acc);
        acc = fmaf(wv.z, xv.z, acc);
        acc = fmaf(wv.w, xv.w, acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) y[row] = acc;
}

// The same product with the row's bytes passing through LDS: a wavefront copies its row, a chunk of whole blocks
// (at most kStageBytes) at a time, with coalesced 16-byte loads into a buffer of its own and decodes from there
// -- the narrow reads of decode4 (two to four bytes each) are then LDS reads instead of vector memory requests
// of a few bytes per lane, which is what bounds matvec_blocks_kernel.  Two buffers: the loads of the next chunk
// are in flight while this one is decoded.  No barriers: a buffer is written and read by one wavefront only,
// whose LDS operations complete in order.  Needs 16-byte aligned rows (row bytes and base pointer).
constexpr int kStageBytes = 4096;

template <int T>
__global__ __launch_bounds__(256) void matvec_blocks_lds_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                                float* __restrict__ y, int n_rows, int k, int chunk_blocks) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    __shared__ __align__(16) uint8_t stage[4][2][kStageBytes];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row = blockIdx.x * 4 + wave;
    if (row >= n_rows) return;
    constexpr int QB = Fmt<T>::kElems / 4, kBytes = Fmt<T>::kBytes;
    const int nblocks = k / Fmt<T>::kElems;
    const uint8_t* rowp = w + (size_t)row * nblocks * kBytes;
    const int nchunks = (nblocks + chunk_blocks - 1) / chunk_blocks;
    u32x4 r[kStageBytes / 1024];
    auto fetch = [&](int c) __attribute__((always_inline)) {
        const int bytes = min(chunk_blocks, nblocks - c * chunk_blocks) * kBytes;
        const uint8_t* src = rowp + (size_t)c * chunk_blocks * kBytes;
#pragma unroll
        for (int u = 0; u < kStageBytes / 1024; u++) {
            const int o = (u * 64 + lane) * 16;
            if (o < bytes) r[u] = *reinterpret_cast<const u32x4*>(src + o);
        }
    };
    fetch(0);
    float acc = 0.f;
    for (int c = 0; c < nchunks; c++) {
        uint8_t* buf = stage[wave][c & 1];
        const int nb_c = min(chunk_blocks, nblocks - c * chunk_blocks), bytes = nb_c * kBytes;
#pragma unroll
        for (int u = 0; u < kStageBytes / 1024; u++) {
            const int o = (u * 64 + lane) * 16;
            if (o < bytes) *reinterpret_cast<u32x4*>(buf + o) = r[u];
        }
        if (c + 1 < nchunks) fetch(c + 1);
        const int nq = nb_c * QB;
        const float4* xq = reinterpret_cast<const float4*>(x) + (size_t)c * chunk_blocks * QB;
        int q = lane;
        for (; q + 64 < nq; q += 128) {
            const float4 w0 = Fmt<T>::decode4(buf + (q / QB) * kBytes, q % QB);
            const float4 w1 = Fmt<T>::decode4(buf + ((q + 64) / QB) * kBytes, (q + 64) % QB);
            const float4 x0 = xq[q], x1 = xq[q + 64];
            acc = fmaf(w0.x, x0.x, acc), acc = fmaf(w0.y, x0.y, acc), acc = fmaf(w0.z, x0.z, acc), acc = fmaf(w0.w, x0.w, acc);
            acc = fmaf(w1.x, x1.x, acc), acc = fmaf(w1.y, x1.y, acc), acc = fmaf(w1.z, x1.z, acc), acc = fmaf(w1.w, x1.w, acc);
        }
        for (; q < nq; q += 64) {
            const float4 wv = Fmt<T>::decode4(buf + (q / QB) * kBytes, q % QB);
            const float4 xv = xq[q];
            acc = fmaf(wv.x, xv.x, acc), acc = fmaf(wv.y, xv.y, acc), acc = fmaf(wv.z, xv.z, acc), acc = fmaf(wv.w, xv.w, acc);
        }
    }
    acc = wave_sum(acc);
    if (lane == 0) y[row] = acc;
}

template <int T>
__global__ __launch_bounds__(256) void matvec_dense_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                           float* __restrict__ y, int n_rows, int k) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n_rows) return;
    const uint8_t* rowp = w + (size_t)row * k * (T == SKN_TYPE_F32 ? 4 : 2);
    float acc = 0.f;
    int done = 0;
    if (T != SKN_TYPE_F32 && (k & 7) == 0 && ((uintptr_t)w & 15) == 0) {
        // eight 16-bit weights per 128-bit load (rows are 16-byte aligned when k is a multiple of 8)
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        for (int o = lane; o < (k >> 3); o += 64) {
            const u32x4 v = reinterpret_cast<const u32x4*>(rowp)[o];
            const float4 x0 = reinterpret_cast<const float4*>(x)[2 * o], x1 = reinterpret_cast<const float4*>(x)[2 * o + 1];
            const uint32_t d[4] = {v.x, v.y, v.z, v.w};
            const float xs8[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float lo = T == SKN_TYPE_F16 ? h2f_bits(d[i] & 0xFFFF) : __uint_as_float(d[i] << 16);
                const float hi = T == SKN_TYPE_F16 ? h2f_bits(d[i] >> 16) : __uint_as_float(d[i] & 0xFFFF0000u);
                acc = fmaf(lo, xs8[2 * i], acc);
                acc = fmaf(hi, xs8[2 * i + 1], acc);
            }
        }
        done = k;
    }
    if (T == SKN_TYPE_F32 && (k & 3) == 0 && ((uintptr_t)w & 15) == 0) {
        // four fp32 weights per 128-bit load, two loads in flight per lane and turn
        const float4* w4 = reinterpret_cast<const float4*>(rowp);
        const float4* x4 = reinterpret_cast<const float4*>(x);
        int o = lane;
        for (; o + 64 < (k >> 2); o += 128) {
            const float4 a0 = w4[o], a1 = w4[o + 64], b0 = x4[o], b1 = x4[o + 64];
            acc = fmaf(a0.x, b0.x, acc), acc = fmaf(a0.y, b0.y, acc), acc = fmaf(a0.z, b0.z, acc), acc = fmaf(a0.w, b0.w, acc);
            acc = fmaf(a1.x, b1.x, acc), acc = fmaf(a1.y, b1.y, acc), acc = fmaf(a1.z, b1.z, acc), acc = fmaf(a1.w, b1.w, acc);
        }
        for (; o < (k >> 2); o += 64) {
            const float4 a0 = w4[o], b0 = x4[o];
            acc = fmaf(a0.x, b0.x, acc), acc = fmaf(a0.y, b0.y, acc), acc = fmaf(a0.z, b0.z, acc), acc = fmaf(a0.w, b0.w, acc);
        }
        done = k;
    }
    for (int i = done + lane; i < k; i += 64) acc = fmaf(dense_at<T>(rowp, i), x[i], acc);
    acc = wave_sum(acc);
    if (lane == 0) y[row] = acc;
}

template <int T>
int launch_dequant(skn_ctx* ctx, const uint8_t* w, int64_t n_elems, float* out) {
    const int64_t n_quads = n_elems / 4, blocks = (n_quads + 255) / 256;
    SKN_REQUIRE(ctx, blocks <= 0x7FFFFFFF, SKN_ERR_SHAPE, "skn_dequant: too many elements for one launch");
    skn_launch(ctx, dequant_blocks_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, w, out, n_quads);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

template <int T>
int launch_convert(skn_ctx* ctx, const uint8_t* w, int64_t n_elems, float* out) {
    const int64_t blocks = (n_elems + 255) / 256;
    SKN_REQUIRE(ctx, blocks <= 0x7FFFFFFF, SKN_ERR_SHAPE, "skn_dequant: too many elements for one launch");
    skn_launch(ctx, convert_dense_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, w, out, n_elems);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

template <int T>
int launch_matvec(skn_ctx* ctx, const uint8_t* w, int n, int k, const float* x, float* y) {
    // whole blocks per chunk, a multiple of the smallest block count whose bytes are a multiple of 16
    constexpr int kBytes = Fmt<T>::kBytes;
    constexpr int kUnit = kBytes % 16 == 0 ? 1 : (kBytes % 8 == 0 ? 2 : (kBytes % 4 == 0 ? 4 : 8));
    const int nblocks = k / Fmt<T>::kElems;
    // Staged where it was measured faster (4096 x 4096 and 4096 x 11008): the formats whose blocks are a multiple of
    // four bytes and read more than a dword and a half-word per quad -- Q5_K twice as fast at k = 11008, Q4_1, Q5_1,
    // Q8_K, IQ4_XS, Q2_K 3-12 %.  In the 18-, 22-, 54-, 66- and 110-byte blocks the dwords straddle LDS banks and
    // the staged kernel is slower (Q5_0: twice), so they keep reading global memory.
    constexpr bool kStaged = kBytes % 4 == 0;
    if (kStaged && nblocks % kUnit == 0 && ((uintptr_t)w & 15) == 0 && ctx->opt_matvec_stage != 0) {
        const int chunk_blocks = kStageBytes / (kUnit * kBytes) * kUnit;
        skn_launch(ctx, matvec_blocks_lds_kernel<T>, dim3((unsigned)((n + 3) / 4)), dim3(256), 0, w, x, y, n, k, chunk_blocks);
        SKN_LAUNCH_CHECK(ctx);
        return SKN_OK;
    }
    skn_launch(ctx, matvec_blocks_kernel<T>, dim3((unsigned)((n + 3) / 4)), dim3(256), 0, w, x, y, n, k);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

template <int T>
int launch_matvec_dense(skn_ctx* ctx, const uint8_t* w, int n, int k, const float* x, float* y) {
    skn_launch(ctx, matvec_dense_kernel<T>, dim3((unsigned)((n + 3) / 4)), dim3(256), 0, w, x, y, n, k);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

template <int T>
int launch_hilo_frag(skn_ctx* ctx, const uint8_t* w, int n, int k, void* bfrag) {
    const dim3 grid((unsigned)(((k >> 6) + kFragChunks - 1) / kFragChunks), (unsigned)((n + 63) / 64 * 2));
    skn_launch(ctx, weights_hilo_frag_kernel<T>, grid, dim3(256), 0, w, (half8_t*)bfrag, n, k);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

}  // namespace

// Internal (arguments already checked by skn_gemm_q; k is a multiple of 64): the weights as the fp16 pair the
// general GEMM path multiplies with, in fragment order; bfrag holds ceil(n / 64) * 64 * k * 4 bytes.
int skn_weights_hilo_frag(skn_ctx* ctx, int ggml_type, const uint8_t* w, int n, int k, void* bfrag) {
    switch (ggml_type) {
        case SKN_TYPE_Q8_0: return launch_hilo_frag<SKN_TYPE_Q8_0>(ctx, w, n, k, bfrag);
        case SKN_TYPE_Q4_K: return launch_hilo_frag<SKN_TYPE_Q4_K>(ctx, w, n, k, bfrag);
        case SKN_TYPE_Q6_K: return launch_hilo_frag<SKN_TYPE_Q6_K>(ctx, w, n, k, bfrag);
        case SKN_TYPE_Q4_0: return launch_hilo_frag<SKN_TYPE_Q4_0>(ctx, w, n, k, bfrag);
        case SKN_TYPE_Q4_1: return launch_hilo_frag<SKN_TYPE_Q4_1>(ctx, w, n, k, bfrag);
        case SKN_TYPE_Q5_0: return launch_hilo_frag<SKN_TYPE_Q5_0>(ctx, w, n, k, bfrag);
        case SKN_TYPE_Q5_1: return launch_hilo_frag<SKN_TYPE_Q5_1>(ctx, w, n, k, bfrag);
        case SKN_TYPE_Q2_K: return launch_hilo_frag<SKN_TYPE_Q2_K>(ctx, w, n, k, bfrag);
        case SKN_TYPE_Q5_K: return launch_hilo_frag<SKN_TYPE_Q5_K>(ctx, w, n, k, bfrag);
        case SKN_TYPE_Q3_K: return launch_hilo_frag<SKN_TYPE_Q3_K>(ctx, w, n, k, bfrag);
        case SKN_TYPE_Q8_K: return launch_hilo_frag<SKN_TYPE_Q8_K>(ctx, w, n, k, bfrag);
        case SKN_TYPE_IQ4_NL: return launch_hilo_frag<SKN_TYPE_IQ4_NL>(ctx, w, n, k, bfrag);
        case SKN_TYPE_IQ4_XS: return launch_hilo_frag<SKN_TYPE_IQ4_XS>(ctx, w, n, k, bfrag);
        case SKN_TYPE_TQ1_0: return launch_hilo_frag<SKN_TYPE_TQ1_0>(ctx, w, n, k, bfrag);
        case SKN_TYPE_TQ2_0: return launch_hilo_frag<SKN_TYPE_TQ2_0>(ctx, w, n, k, bfrag);
        case SKN_TYPE_F32: return launch_hilo_frag<SKN_TYPE_F32>(ctx, w, n, k, bfrag);
        case SKN_TYPE_F16: return launch_hilo_frag<SKN_TYPE_F16>(ctx, w, n, k, bfrag);
        case SKN_TYPE_BF16: return launch_hilo_frag<SKN_TYPE_BF16>(ctx, w, n, k, bfrag);
        default: return skn_fail(ctx, SKN_ERR_TYPE, "skn_gemm_q: ggml type %d is not supported", ggml_type);
    }
}


// Called by skn_dequant / skn_matvec_q after their argument checks, for the types they do not handle themselves.
int skn_dequant_other(skn_ctx* ctx, int ggml_type, const uint8_t* w, int64_t n_elems, float* out) {
    switch (ggml_type) {
        case SKN_TYPE_Q4_0: return launch_dequant<SKN_TYPE_Q4_0>(ctx, w, n_elems, out);
        case SKN_TYPE_Q4_1: return launch_dequant<SKN_TYPE_Q4_1>(ctx, w, n_elems, out);
        case SKN_TYPE_Q5_0: return launch_dequant<SKN_TYPE_Q5_0>(ctx, w, n_elems, out);
        case SKN_TYPE_Q5_1: return launch_dequant<SKN_TYPE_Q5_1>(ctx, w, n_elems, out);
        case SKN_TYPE_Q2_K: return launch_dequant<SKN_TYPE_Q2_K>(ctx, w, n_elems, out);
        case SKN_TYPE_Q5_K: return launch_dequant<SKN_TYPE_Q5_K>(ctx, w, n_elems, out);
        case SKN_TYPE_Q3_K: return launch_dequant<SKN_TYPE_Q3_K>(ctx, w, n_elems, out);
        case SKN_TYPE_Q8_K: return launch_dequant<SKN_TYPE_Q8_K>(ctx, w, n_elems, out);
        case SKN_TYPE_IQ4_NL: return launch_dequant<SKN_TYPE_IQ4_NL>(ctx, w, n_elems, out);
        case SKN_TYPE_IQ4_XS: return launch_dequant<SKN_TYPE_IQ4_XS>(ctx, w, n_elems, out);
        case SKN_TYPE_TQ1_0: return launch_dequant<SKN_TYPE_TQ1_0>(ctx, w, n_elems, out);
        case SKN_TYPE_TQ2_0: return launch_dequant<SKN_TYPE_TQ2_0>(ctx, w, n_elems, out);
        case SKN_TYPE_F32: return launch_convert<SKN_TYPE_F32>(ctx, w, n_elems, out);
        case SKN_TYPE_F16: return launch_convert<SKN_TYPE_F16>(ctx, w, n_elems, out);
        case SKN_TYPE_BF16: return launch_convert<SKN_TYPE_BF16>(ctx, w, n_elems, out);
        default: return skn_fail(ctx, SKN_ERR_TYPE, "skn_dequant: ggml type %d is not supported", ggml_type);
    }
}

int skn_matvec_other(skn_ctx* ctx, int ggml_type, const uint8_t* w, int n, int k, const float* x, float* y) {
    switch (ggml_type) {
        case SKN_TYPE_Q4_0: return launch_matvec<SKN_TYPE_Q4_0>(ctx, w, n, k, x, y);
        case SKN_TYPE_Q4_1: return launch_matvec<SKN_TYPE_Q4_1>(ctx, w, n, k, x, y);
        case SKN_TYPE_Q5_0: return launch_matvec<SKN_TYPE_Q5_0>(ctx, w, n, k, x, y);
        case SKN_TYPE_Q5_1: return launch_matvec<SKN_TYPE_Q5_1>(ctx, w, n, k, x, y);
        case SKN_TYPE_Q2_K: return launch_matvec<SKN_TYPE_Q2_K>(ctx, w, n, k, x, y);
        case SKN_TYPE_Q5_K: return launch_matvec<SKN_TYPE_Q5_K>(ctx, w, n, k, x, y);
        case SKN_TYPE_Q3_K: return launch_matvec<SKN_TYPE_Q3_K>(ctx, w, n, k, x, y);
        case SKN_TYPE_Q8_K: return launch_matvec<SKN_TYPE_Q8_K>(ctx, w, n, k, x, y);
        case SKN_TYPE_IQ4_NL: return launch_matvec<SKN_TYPE_IQ4_NL>(ctx, w, n, k, x, y);
        case SKN_TYPE_IQ4_XS: return launch_matvec<SKN_TYPE_IQ4_XS>(ctx, w, n, k, x, y);
        case SKN_TYPE_TQ1_0: return launch_matvec<SKN_TYPE_TQ1_0>(ctx, w, n, k, x, y);
        case SKN_TYPE_TQ2_0: return launch_matvec<SKN_TYPE_TQ2_0>(ctx, w, n, k, x, y);
        case SKN_TYPE_F32: return launch_matvec_dense<SKN_TYPE_F32>(ctx, w, n, k, x, y);
        case SKN_TYPE_F16: return launch_matvec_dense<SKN_TYPE_F16>(ctx, w, n, k, x, y);
        case SKN_TYPE_BF16: return launch_matvec_dense<SKN_TYPE_BF16>(ctx, w, n, k, x, y);
        default: return skn_fail(ctx, SKN_ERR_TYPE, "skn_matvec_q: ggml type %d is not supported", ggml_type);
    }
}
