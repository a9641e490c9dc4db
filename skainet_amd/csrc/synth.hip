// Seeded synthetic inputs of the benchmark shapes, generated on the host by the library itself so that every harness
// above the C ABI (C, ctypes, a Kotlin binding) draws identical bytes.  Integer arithmetic only up to the final
// conversions: the same seed gives the same buffer on every machine and in every restatement (skainet_amd/synth.py
// holds one in NumPy; tests compare the two byte for byte).
//
//   word(seed, stream, i) = mix(mix(seed + G * (stream + 1)) + G * (i + 1)),  G = 0x9E3779B97F4A7C15,
//   mix = the SplitMix64 finalizer.  Counter-based: any element can be produced on its own.
//   bytes:   word j of a stream gives bytes 8j .. 8j+7, least significant first.
//   normal:  element i of a stream is (sum of the twelve 32-bit halves of words 6i .. 6i+5 - 6 * 2^32) / 2^32 --
//            the sum of twelve uniforms minus six (mean 0, variance 1, |value| <= 6), exact in double.
//   streams: 0 quants / plain values, 1 d, 2 dmin, 3 scales and mins.
// Block contents follow BASELINE's recipe (gguf/src/commonMain/kotlin/sk/ai/net/gguf/Constants.kt:65,69,71 pins the
// sizes): Q8_0 d = f16(|N| * 0.02), quants uniform in [-127, 127]; Q4_K d = f16(|N| * 0.01), dmin = f16(|N| * 0.005),
// sixteen 6-bit scales / mins uniform in 0..63, nibbles uniform; Q6_K 6-bit quants uniform, int8 scales uniform in
// [-32, 31], d = f16(|N| * 0.01).  Conversions to fp16 / bf16 go through fp32 and round to nearest even.
#include "common.h"

namespace {

constexpr uint64_t kG = 0x9E3779B97F4A7C15ull;

inline uint64_t mix(uint64_t z) {
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

struct Stream {
    uint64_t base;
    Stream(uint64_t seed, int stream) : base(mix(seed + kG * (uint64_t)(stream + 1))) {}
    uint64_t word(uint64_t i) const { return mix(base + kG * (i + 1)); }
    void bytes(uint64_t first_word, uint8_t* out, size_t n) const {
        for (size_t j = 0; j < n; j += 8) {
            const uint64_t w = word(first_word + j / 8);
            for (size_t b = 0; b < 8 && j + b < n; b++) out[j + b] = (uint8_t)(w >> (8 * b));
        }
    }
    double normal(uint64_t i) const {
        uint64_t sum = 0;
        for (int j = 0; j < 6; j++) {
            const uint64_t w = word(6 * i + j);
            sum += (w & 0xFFFFFFFFull) + (w >> 32);
        }
        return ((double)(int64_t)(sum - (6ull << 32))) * (1.0 / 4294967296.0);
    }
};

uint16_t f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    x &= 0x7FFFFFFFu;
    if (x >= 0x7F800000u) return (uint16_t)(sign | 0x7C00u | (x > 0x7F800000u ? 0x200u : 0u));
    if (x >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);  // rounds to infinity
    if (x < 0x33000001u) return (uint16_t)sign;               // rounds to zero
    const int e = (int)(x >> 23) - 127;
    uint32_t m = (x & 0x7FFFFFu) | 0x800000u;
    int shift = e >= -14 ? 13 : 13 + (-14 - e);               // bits dropped from the 24-bit significand
    uint32_t h = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (h & 1))) h++;
    // h carries the hidden bit for normal results (e >= -14): (h - 0x400) + ((e + 15) << 10); a carry out of the
    // significand moves into the exponent field by itself
    return (uint16_t)(sign | (e >= -14 ? h + ((uint32_t)(e + 14) << 10) : h));
}

uint16_t f32_to_bf16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    return (uint16_t)((x + 0x7FFFu + ((x >> 16) & 1u)) >> 16);
}

inline void put_f16(uint8_t* p, double v) {
    const uint16_t h = f32_to_f16((float)v);
    p[0] = (uint8_t)h;
    p[1] = (uint8_t)(h >> 8);
}

}  // namespace

extern "C" int skn_synth_weight(int ggml_type, int64_t n_rows, int64_t k, uint64_t seed, void* host_out, size_t out_bytes) {
    SKN_REQUIRE(nullptr, ggml_type == SKN_TYPE_Q8_0 || ggml_type == SKN_TYPE_Q4_K || ggml_type == SKN_TYPE_Q6_K, SKN_ERR_TYPE,
                "skn_synth_weight: ggml type %d has no generator (Q8_0, Q4_K, Q6_K)", ggml_type);
    int be = 0, bb = 0;
    skn_type_block(ggml_type, &be, &bb);
    SKN_REQUIRE(nullptr, n_rows >= 0 && k >= 0, SKN_ERR_ARG, "skn_synth_weight: negative shape");
    SKN_REQUIRE(nullptr, k % be == 0, SKN_ERR_SHAPE, "Quantized tensor row size (%lld) is not a multiple of block size (%d)",
                (long long)k, be);
    const uint64_t nblocks = (uint64_t)n_rows * (uint64_t)(k / be);
    SKN_REQUIRE(nullptr, out_bytes == nblocks * (uint64_t)bb, SKN_ERR_SHAPE, "skn_synth_weight: the buffer holds %zu bytes, the weight %llu",
                out_bytes, (unsigned long long)(nblocks * (uint64_t)bb));
    if (nblocks == 0) return SKN_OK;
    SKN_REQUIRE(nullptr, host_out != nullptr, SKN_ERR_ARG, "skn_synth_weight: null buffer");
    const Stream q(seed, 0), d(seed, 1), dmin(seed, 2), sc(seed, 3);
    uint8_t* out = (uint8_t*)host_out;
    for (uint64_t b = 0; b < nblocks; b++) {
        uint8_t* blk = out + b * (uint64_t)bb;
        if (ggml_type == SKN_TYPE_Q8_0) {
            put_f16(blk, fabs(d.normal(b)) * 0.02);
            uint8_t raw[64];
            q.bytes(8 * b, raw, 64);
            for (int i = 0; i < 32; i++) {
                const uint32_t u = (uint32_t)raw[2 * i] | ((uint32_t)raw[2 * i + 1] << 8);
                blk[2 + i] = (uint8_t)(int8_t)((int)((u * 255u) >> 16) - 127);
            }
        } else if (ggml_type == SKN_TYPE_Q4_K) {
            put_f16(blk, fabs(d.normal(b)) * 0.01);
            put_f16(blk + 2, fabs(dmin.normal(b)) * 0.005);
            uint8_t v[16];  // scales of the eight sub-blocks, then their mins
            sc.bytes(2 * b, v, 16);
            for (int i = 0; i < 16; i++) v[i] &= 63;
            for (int j = 0; j < 4; j++) {
                blk[4 + j] = (uint8_t)(v[j] | ((v[4 + j] >> 4) << 6));
                blk[8 + j] = (uint8_t)(v[8 + j] | ((v[12 + j] >> 4) << 6));
                blk[12 + j] = (uint8_t)((v[4 + j] & 0x0F) | ((v[12 + j] & 0x0F) << 4));
            }
            q.bytes(16 * b, blk + 16, 128);
        } else {
            q.bytes(24 * b, blk, 192);
            uint8_t v[16];
            sc.bytes(2 * b, v, 16);
            for (int i = 0; i < 16; i++) blk[192 + i] = (uint8_t)(int8_t)((int)(v[i] & 63) - 32);
            put_f16(blk + 208, fabs(d.normal(b)) * 0.01);
        }
    }
    return SKN_OK;
}

extern "C" int skn_synth_activation_f32(int64_t n, uint64_t seed, float* host_out) {
    SKN_REQUIRE(nullptr, n >= 0 && (n == 0 || host_out), SKN_ERR_ARG, "skn_synth_activation_f32: bad arguments");
    const Stream s(seed, 0);
    for (int64_t i = 0; i < n; i++) host_out[i] = (float)s.normal((uint64_t)i);
    return SKN_OK;
}

extern "C" int skn_synth_activation_bf16(int64_t n, uint64_t seed, uint16_t* host_out) {
    SKN_REQUIRE(nullptr, n >= 0 && (n == 0 || host_out), SKN_ERR_ARG, "skn_synth_activation_bf16: bad arguments");
    const Stream s(seed, 0);
    for (int64_t i = 0; i < n; i++) host_out[i] = f32_to_bf16((float)s.normal((uint64_t)i));
    return SKN_OK;
}

extern "C" int skn_synth_kv_f16(int64_t n, uint64_t seed, uint16_t* host_out) {
    SKN_REQUIRE(nullptr, n >= 0 && (n == 0 || host_out), SKN_ERR_ARG, "skn_synth_kv_f16: bad arguments");
    const Stream s(seed, 0);
    for (int64_t i = 0; i < n; i++) host_out[i] = f32_to_f16((float)s.normal((uint64_t)i));
    return SKN_OK;
}

extern "C" uint64_t skn_synth_checksum(const void* host, size_t bytes) {
    uint64_t h = 0xCBF29CE484222325ull;  // FNV-1a 64 over every byte
    const uint8_t* p = (const uint8_t*)host;
    for (size_t i = 0; i < bytes; i++) h = (h ^ p[i]) * 0x100000001B3ull;
    return h;
}
