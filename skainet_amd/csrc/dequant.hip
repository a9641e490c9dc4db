// GGUF block dequantization (Q8_0, Q4_K, Q6_K) -> fp32, bit-exact with the ggml block formulas.
//
// Every thread produces four consecutive fp32 outputs (one 16-byte store), so a wavefront writes 1 KiB
// contiguous per store instruction; the kernels are bound by the fp32 write stream (4 B per element out
// against 0.56-1.06 B per element in).  Products are formed with the explicitly rounded intrinsics so that
// no contraction can change a bit: each value is the exact real d*sc*q (- dmin*m) rounded once.
#include "common.h"

namespace {

// Q8_0: 34-byte block = f16 d @0, int8 qs[32] @2.
__global__ __launch_bounds__(256) void dequant_q8_0_kernel(const uint8_t* __restrict__ w, float* __restrict__ out,
                                                           int64_t n_quads) {
    int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_quads) return;
    int64_t blk = t >> 3;   // 8 quads of 4 elements per 32-element block
    int quad = (int)(t & 7);
    const uint8_t* b = w + blk * 34;
    float d = h2f_bits(load_u16_a2(b));
    uint32_t q = load_u32_a2(b + 2 + 4 * quad);
    float4 y;
    y.x = __fmul_rn(d, (float)(int8_t)(q & 0xFF));
    y.y = __fmul_rn(d, (float)(int8_t)((q >> 8) & 0xFF));
    y.z = __fmul_rn(d, (float)(int8_t)((q >> 16) & 0xFF));
    y.w = __fmul_rn(d, (float)(int8_t)(q >> 24));
    reinterpret_cast<float4*>(out)[t] = y;
}

// Q4_K: 144-byte superblock = f16 d @0, f16 dmin @2, 12 packed 6-bit scale/min bytes @4, 128 nibble bytes @16.
// A thread takes one dword of nibbles and writes both of its quads -- the low nibbles (elements 64c + r .. + 3 of
// sub-block 2c) and the high ones (the same positions of sub-block 2c + 1, 32 elements on): 32 threads per
// superblock, one header load and one nibble load for two 16-byte stores; eight consecutive lanes still write one
// whole 128-byte line per store.
__global__ __launch_bounds__(256) void dequant_q4_k_kernel(const uint8_t* __restrict__ w, float* __restrict__ out,
                                                           int64_t n_pairs) {
    int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_pairs) return;
    int64_t blk = t >> 5;        // 32 quad pairs per 256-element superblock
    const int u = (int)(t & 31);
    const int c = u >> 3, r = (u & 7) * 4;  // 64-element chunk, first position in its low half
    // superblocks are 16-byte aligned: the whole header (d, dmin, twelve scale / min bytes) is one 128-bit load
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const u32x4* b128 = reinterpret_cast<const u32x4*>(w + blk * 144);
    const u32x4 hdr = b128[0];
    const float d = h2f_bits(hdr.x & 0xFFFF), dmin = h2f_bits(hdr.x >> 16);
    // bytes 0..3 of the twelve: low scales, 4..7: low mins, 8..11: low nibbles of the high ones, whose top two
    // bits sit in bits 6..7 of the first eight bytes.  Sub-blocks j = 2c (low nibbles) and 2c + 1 (high nibbles)
    int sc[2], m[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int j = 2 * c + i, sh = 8 * (j & 3);
        if (j < 4) {
            sc[i] = (hdr.y >> sh) & 63;
            m[i] = (hdr.z >> sh) & 63;
        } else {
            sc[i] = ((hdr.w >> sh) & 0x0F) | (((hdr.y >> (sh + 6)) & 3) << 4);
            m[i] = ((hdr.w >> (sh + 4)) & 0x0F) | (((hdr.z >> (sh + 6)) & 3) << 4);
        }
    }
    const uint32_t q = reinterpret_cast<const uint32_t*>(b128)[4 + 8 * c + (r >> 2)];
    float4* dst = reinterpret_cast<float4*>(out + blk * 256 + 64 * c + r);
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const uint32_t qq = q >> (4 * i);
        const float d1 = __fmul_rn(d, (float)sc[i]);
        const float m1 = __fmul_rn(dmin, (float)m[i]);
        float4 y;
        y.x = __fsub_rn(__fmul_rn(d1, (float)(qq & 0xF)), m1);
        y.y = __fsub_rn(__fmul_rn(d1, (float)((qq >> 8) & 0xF)), m1);
        y.z = __fsub_rn(__fmul_rn(d1, (float)((qq >> 16) & 0xF)), m1);
        y.w = __fsub_rn(__fmul_rn(d1, (float)((qq >> 24) & 0xF)), m1);
        dst[8 * i] = y;  // + 32 elements
    }
}

// Q6_K: 210-byte superblock = ql[128] @0 (low nibbles), qh[64] @128 (high bit pairs), int8 scales[16] @192, f16 d @208.
// A thread takes one dword of ql and the dword of qh that goes with it and writes both quads that share them: the
// low nibbles (quarter p = 0 or 1 of half n) and the high nibbles (quarter p + 2, 64 elements on).
__global__ __launch_bounds__(256) void dequant_q6_k_kernel(const uint8_t* __restrict__ w, float* __restrict__ out,
                                                           int64_t n_pairs) {
    int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_pairs) return;
    int64_t blk = t >> 5;
    const int u = (int)(t & 31);
    const uint8_t* b = w + blk * 210;  // only 2-byte aligned
    const int n = u >> 4, p = (u >> 3) & 1, l = (u & 7) * 4;
    const uint32_t lo = load_u32_a2(b + 64 * n + 32 * p + l);
    const uint32_t hi = load_u32_a2(b + 128 + 32 * n + l);
    const float d = h2f_bits(load_u16_a2(b + 208));
    float4* dst = reinterpret_cast<float4*>(out + blk * 256 + 128 * n + 32 * p + l);
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int quarter = p + 2 * i;
        const uint32_t lq = lo >> (4 * i), hq = hi >> (2 * quarter);
        const float sc = (float)(int8_t)b[192 + 8 * n + 2 * quarter + (l >> 4)];
        const float ds = __fmul_rn(d, sc);
        float4 y;
        y.x = __fmul_rn(ds, (float)((int)((lq & 0xF) | ((hq & 3) << 4)) - 32));
        y.y = __fmul_rn(ds, (float)((int)(((lq >> 8) & 0xF) | (((hq >> 8) & 3) << 4)) - 32));
        y.z = __fmul_rn(ds, (float)((int)(((lq >> 16) & 0xF) | (((hq >> 16) & 3) << 4)) - 32));
        y.w = __fmul_rn(ds, (float)((int)(((lq >> 24) & 0xF) | (((hq >> 24) & 3) << 4)) - 32));
        dst[16 * i] = y;  // + 64 elements
    }
}

}  // namespace

extern "C" int skn_dequant(skn_ctx* ctx, int ggml_type, const void* w_dev, int64_t n_elems, float* out_dev) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_dequant: ctx is null");
    SKN_REQUIRE(ctx, skn_is_quant(ggml_type), SKN_ERR_TYPE, "skn_dequant: ggml type %d is not supported", ggml_type);
    int be, bb;
    skn_type_block(ggml_type, &be, &bb);
    SKN_REQUIRE(ctx, n_elems >= 0 && n_elems % be == 0, SKN_ERR_SHAPE,
                "skn_dequant: element count (%lld) is not a multiple of block size (%d)", (long long)n_elems, be);
    if (n_elems == 0) return SKN_OK;
    SKN_REQUIRE(ctx, w_dev && out_dev, SKN_ERR_ARG, "skn_dequant: null pointer");
    SKN_REQUIRE(ctx, ((uintptr_t)out_dev & 15) == 0, SKN_ERR_ARG, "skn_dequant: out must be 16-byte aligned");
    SKN_REQUIRE(ctx, ((uintptr_t)w_dev & (ggml_type == SKN_TYPE_Q4_K ? 15 : ggml_type == SKN_TYPE_F32 ? 3 : 1)) == 0,
                SKN_ERR_ARG, "skn_dequant: weight pointer is misaligned for its block type");
    if (!skn_is_core_quant(ggml_type)) return skn_dequant_other(ctx, ggml_type, (const uint8_t*)w_dev, n_elems, out_dev);
    int64_t n_quads = n_elems / 4;
    int64_t blocks = (n_quads + 255) / 256;
    SKN_REQUIRE(ctx, blocks <= 0x7FFFFFFF, SKN_ERR_SHAPE, "skn_dequant: too many elements for one launch");
    const uint8_t* w = (const uint8_t*)w_dev;
    dim3 grid((unsigned)blocks), block(256);
    if (ggml_type == SKN_TYPE_Q8_0)
        skn_launch(ctx, dequant_q8_0_kernel, grid, block, 0, w, out_dev, n_quads);
    else if (ggml_type == SKN_TYPE_Q4_K)
        skn_launch(ctx, dequant_q4_k_kernel, dim3((unsigned)((n_quads / 2 + 255) / 256)), block, 0, w, out_dev, n_quads / 2);
    else
        skn_launch(ctx, dequant_q6_k_kernel, dim3((unsigned)((n_quads / 2 + 255) / 256)), block, 0, w, out_dev, n_quads / 2);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}
