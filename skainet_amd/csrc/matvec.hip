// Batch-1 quantized matvec  y[n] = sum_k deq(W)[n,k] * x[k]  for GGUF Q4_K, Q8_0 and Q6_K weights.
//
// The op is bound by the HBM read of the weight blocks (0.5625 / 1.0625 / 0.8203 bytes per weight); x is
// read once per workgroup and y written once.  One wavefront owns one output row, so the only cross-lane
// traffic is a single DPP reduction per row and rows never need atomics.
#include "common.h"

namespace {

// ------------------------------------------------------------------------------------------ Q4_K
//
// A row of k weights is k/256 superblocks of 144 bytes = 9 aligned 16-byte chunks each: one header chunk
// (f16 d, f16 dmin, 12 bytes of 6-bit scales/mins) and eight chunks of nibbles.  Per step a wavefront takes
// eight superblocks: lane (b, c) = (lane / 8, lane % 8) loads nibble chunk c of superblock b with one
// 128-bit load (64 lanes x 16 B, eight 128-byte runs) and the superblock's header with a second 128-bit load
// that its eight lanes share.  All loads of a row are issued before anything is consumed, so a row's whole
// byte range is in flight at once.
//
// Nibble chunk c holds bytes 16c..16c+15 of qs: low nibbles are elements 64*(c/2) + 16*(c%2) + 0..15 (sub-block
// 2*(c/2)), high nibbles the same positions + 32 (sub-block 2*(c/2)+1).  The activation is staged in LDS in
// exactly that lane order -- slot [(step*8 + i)*64 + lane] holds the i-th float4 the lane needs -- so the
// eight 128-bit LDS reads of a step are conflict-free, together with the two 16-element partial sums of x
// that the "- dmin * m" term needs.
//
//   y += d * (sc_lo * sum(q_lo * x_lo) + sc_hi * sum(q_hi * x_hi)) - dmin * (m_lo * sum(x_lo) + m_hi * sum(x_hi))

constexpr int kQ4kBlockBytes = 144;

__device__ __forceinline__ void q4k_pair_scales(const uint4& h, int pair, float& sc0, float& sc1, float& m0,
                                                float& m1) {
    // pair p covers sub-blocks 2p and 2p+1; scales[] = bytes of (h.y, h.z, h.w)
    const int sh = 16 * (pair & 1);
    const uint32_t a = (h.y >> sh) & 0xFFFF;  // scales[j], scales[j+1] of the low group (j = 2p or 2p-4)
    const uint32_t b = (h.z >> sh) & 0xFFFF;  // scales[4+..]
    const uint32_t c = (h.w >> sh) & 0xFFFF;  // scales[8+..]
    uint32_t s0, s1, n0, n1;
    if (pair < 2) {
        s0 = a & 63;
        s1 = (a >> 8) & 63;
        n0 = b & 63;
        n1 = (b >> 8) & 63;
    } else {
        s0 = (c & 0xF) | (((a >> 6) & 3) << 4);
        s1 = ((c >> 8) & 0xF) | (((a >> 14) & 3) << 4);
        n0 = ((c >> 4) & 0xF) | (((b >> 6) & 3) << 4);
        n1 = ((c >> 12) & 0xF) | (((b >> 14) & 3) << 4);
    }
    sc0 = (float)s0;
    sc1 = (float)s1;
    m0 = (float)n0;
    m1 = (float)n1;
}

// sum over the 4 bytes of q of nibble * x: low nibbles against xl, high nibbles against xh
__device__ __forceinline__ void q4k_dot_dword(uint32_t q, const float4& xl, const float4& xh, float& alo, float& ahi) {
    const uint32_t lo = q & 0x0F0F0F0Fu;
    const uint32_t hi = (q >> 4) & 0x0F0F0F0Fu;
    alo = fmaf((float)(lo & 0xFF), xl.x, alo);
    alo = fmaf((float)((lo >> 8) & 0xFF), xl.y, alo);
    alo = fmaf((float)((lo >> 16) & 0xFF), xl.z, alo);
    alo = fmaf((float)(lo >> 24), xl.w, alo);
    ahi = fmaf((float)(hi & 0xFF), xh.x, ahi);
    ahi = fmaf((float)((hi >> 8) & 0xFF), xh.y, ahi);
    ahi = fmaf((float)((hi >> 16) & 0xFF), xh.z, ahi);
    ahi = fmaf((float)(hi >> 24), xh.w, ahi);
}

// Stage x for Q4_K rows of nb superblocks into LDS in lane order; see the layout note above.
__device__ __forceinline__ void q4k_stage_x(const float* __restrict__ x, int nb, float4* xs, float2* ss, int tid,
                                            int nthreads) {
    const int ncols = nb * 8;  // one column of 32 activations per (superblock, nibble chunk)
    const int steps = (nb + 7) >> 3;
    for (int cc = tid; cc < steps * 64; cc += nthreads) {
        const int step = cc >> 6, lane = cc & 63;
        float4 v[8];
        if (cc < ncols) {
            const int blk = cc >> 3, c = cc & 7;
            const float4* src = reinterpret_cast<const float4*>(x + 256 * blk + 64 * (c >> 1) + 16 * (c & 1));
#pragma unroll
            for (int i = 0; i < 4; i++) {
                v[i] = src[i];
                v[4 + i] = src[8 + i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
        float slo = 0.f, shi = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            slo += (v[i].x + v[i].y) + (v[i].z + v[i].w);
            shi += (v[4 + i].x + v[4 + i].y) + (v[4 + i].z + v[4 + i].w);
        }
#pragma unroll
        for (int i = 0; i < 8; i++) xs[(step * 8 + i) * 64 + lane] = v[i];
        ss[cc] = make_float2(slo, shi);
    }
}

// STEPS > 0: the row is covered by exactly STEPS fully unrolled steps with every load hoisted.
// STEPS == 0: generic rolled loop for any k.
template <int STEPS>
__global__ __launch_bounds__(1024) void matvec_q4k_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                          float* __restrict__ y, int n_rows, int nb) {
    extern __shared__ float4 lds4[];
    const int steps = STEPS > 0 ? STEPS : (nb + 7) >> 3;
    float4* xs = lds4;
    float2* ss = reinterpret_cast<float2*>(lds4 + steps * 8 * 64);

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int waves = blockDim.x >> 6;
    const int row = blockIdx.x * waves + wave;
    const bool row_ok = row < n_rows;
    const int sub = lane >> 3;  // superblock within the step
    const int c = lane & 7;     // nibble chunk within the superblock
    const uint4* rowp = reinterpret_cast<const uint4*>(w + (size_t)(row_ok ? row : 0) * nb * kQ4kBlockBytes);

    if constexpr (STEPS > 0) {
        uint4 qv[STEPS], hv[STEPS];
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            const int blk = s * 8 + sub;
            const bool ok = row_ok && blk < nb;
            const uint4* bp = rowp + (ok ? blk : 0) * 9;
            qv[s] = bp[1 + c];
            hv[s] = bp[0];
            if (!ok) {
                qv[s] = make_uint4(0, 0, 0, 0);
                hv[s] = make_uint4(0, 0, 0, 0);
            }
        }
        q4k_stage_x(x, nb, xs, ss, threadIdx.x, blockDim.x);
        __syncthreads();
        float acc = 0.f;
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            float alo = 0.f, ahi = 0.f;
            const uint32_t q[4] = {qv[s].x, qv[s].y, qv[s].z, qv[s].w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float4 xl = xs[(s * 8 + i) * 64 + lane];
                const float4 xh = xs[(s * 8 + 4 + i) * 64 + lane];
                q4k_dot_dword(q[i], xl, xh, alo, ahi);
            }
            const float2 sx = ss[s * 64 + lane];
            float sc0, sc1, m0, m1;
            q4k_pair_scales(hv[s], c >> 1, sc0, sc1, m0, m1);
            const float d = h2f_bits(hv[s].x & 0xFFFF), dmin = h2f_bits(hv[s].x >> 16);
            acc += d * (sc0 * alo + sc1 * ahi) - dmin * (m0 * sx.x + m1 * sx.y);
        }
        acc = wave_sum(acc);
        if (row_ok && lane == 0) y[row] = acc;
    } else {
        q4k_stage_x(x, nb, xs, ss, threadIdx.x, blockDim.x);
        __syncthreads();
        float acc = 0.f;
        for (int s = 0; s < steps; s++) {
            const int blk = s * 8 + sub;
            if (row_ok && blk < nb) {
                const uint4* bp = rowp + blk * 9;
                const uint4 qq = bp[1 + c];
                const uint4 hh = bp[0];
                float alo = 0.f, ahi = 0.f;
                const uint32_t q[4] = {qq.x, qq.y, qq.z, qq.w};
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float4 xl = xs[(s * 8 + i) * 64 + lane];
                    const float4 xh = xs[(s * 8 + 4 + i) * 64 + lane];
                    q4k_dot_dword(q[i], xl, xh, alo, ahi);
                }
                const float2 sx = ss[s * 64 + lane];
                float sc0, sc1, m0, m1;
                q4k_pair_scales(hh, c >> 1, sc0, sc1, m0, m1);
                const float d = h2f_bits(hh.x & 0xFFFF), dmin = h2f_bits(hh.x >> 16);
                acc += d * (sc0 * alo + sc1 * ahi) - dmin * (m0 * sx.x + m1 * sx.y);
            }
        }
        acc = wave_sum(acc);
        if (row_ok && lane == 0) y[row] = acc;
    }
}

// ------------------------------------------------------------------------------------------ Q8_0
//
// 34-byte blocks (f16 d, 32 x int8), only 2-byte aligned.  One wavefront per row; lane l takes blocks
// l, l+64, ...  The lane's 34 bytes are fetched as seventeen 16-bit loads (consecutive lanes read
// consecutive blocks, so the wavefront still walks one contiguous range) and x as eight aligned float4.
__global__ __launch_bounds__(256) void matvec_q8_0_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                          float* __restrict__ y, int n_rows, int nb) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= n_rows) return;
    const uint8_t* rowp = w + (size_t)row * nb * 34;
    float acc = 0.f;
    for (int blk = lane; blk < nb; blk += 64) {
        const uint16_t* b16 = reinterpret_cast<const uint16_t*>(rowp + (size_t)blk * 34);
        const float d = h2f_bits(b16[0]);
        const float4* xp = reinterpret_cast<const float4*>(x + 32 * blk);
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t q = (uint32_t)b16[1 + 2 * i] | ((uint32_t)b16[2 + 2 * i] << 16);
            const float4 xv = xp[i];
            s = fmaf((float)(int8_t)(q & 0xFF), xv.x, s);
            s = fmaf((float)(int8_t)((q >> 8) & 0xFF), xv.y, s);
            s = fmaf((float)(int8_t)((q >> 16) & 0xFF), xv.z, s);
            s = fmaf((float)(int8_t)(q >> 24), xv.w, s);
        }
        acc = fmaf(d, s, acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) y[row] = acc;
}

// ------------------------------------------------------------------------------------------ Q6_K
//
// 210-byte superblocks, 2-byte aligned.  One wavefront per row, one superblock per step: lane (n, l) =
// (lane / 32, lane % 32) owns the four elements 128n + l + {0, 32, 64, 96}, which share the bytes
// ql[64n + l], ql[64n + l + 32] and qh[32n + l]; the 64 lanes read 64 consecutive bytes per load.
__global__ __launch_bounds__(256) void matvec_q6_k_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                          float* __restrict__ y, int n_rows, int nb) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= n_rows) return;
    const uint8_t* rowp = w + (size_t)row * nb * 210;
    const int n = lane >> 5, l = lane & 31;
    float acc = 0.f;
    for (int blk = 0; blk < nb; blk++) {
        const uint8_t* b = rowp + (size_t)blk * 210;
        const uint32_t la = b[64 * n + l], lb = b[64 * n + l + 32], h = b[128 + 32 * n + l];
        const int8_t* sc = reinterpret_cast<const int8_t*>(b + 192 + 8 * n + (l >> 4));
        const float d = h2f_bits(load_u16_a2(b + 208));
        const float* xp = x + 256 * blk + 128 * n + l;
        const float q1 = (float)((int)((la & 0xF) | ((h & 3) << 4)) - 32);
        const float q2 = (float)((int)((lb & 0xF) | (((h >> 2) & 3) << 4)) - 32);
        const float q3 = (float)((int)((la >> 4) | (((h >> 4) & 3) << 4)) - 32);
        const float q4 = (float)((int)((lb >> 4) | (((h >> 6) & 3) << 4)) - 32);
        float s = (float)sc[0] * q1 * xp[0];
        s = fmaf((float)sc[2] * q2, xp[32], s);
        s = fmaf((float)sc[4] * q3, xp[64], s);
        s = fmaf((float)sc[6] * q4, xp[96], s);
        acc = fmaf(d, s, acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) y[row] = acc;
}

template <int STEPS>
int launch_q4k(skn_ctx* ctx, const uint8_t* w, int n, int nb, const float* x, float* y, int waves) {
    const int steps = STEPS > 0 ? STEPS : (nb + 7) / 8;
    const size_t lds = (size_t)steps * 64 * (8 * sizeof(float4) + sizeof(float2));
    SKN_REQUIRE(ctx, lds <= 160 * 1024, SKN_ERR_SHAPE, "skn_matvec_q: k = %d needs %zu bytes of LDS (limit 163840)",
                nb * 256, lds);
    auto kern = matvec_q4k_kernel<STEPS>;
    if (lds > 48 * 1024)
        SKN_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                         (int)lds));
    dim3 grid((unsigned)((n + waves - 1) / waves)), block((unsigned)(waves * 64));
    skn_launch(ctx, kern, grid, block, lds, w, x, y, n, nb);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

}  // namespace

extern "C" int skn_matvec_q(skn_ctx* ctx, int ggml_type, const void* w_dev, int n, int k, const float* x_dev,
                            float* y_dev) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_matvec_q: ctx is null");
    SKN_REQUIRE(ctx, skn_is_quant(ggml_type), SKN_ERR_TYPE, "skn_matvec_q: ggml type %d is not supported", ggml_type);
    SKN_REQUIRE(ctx, n >= 0 && k >= 0, SKN_ERR_ARG, "skn_matvec_q: negative shape");
    int be, bb;
    skn_type_block(ggml_type, &be, &bb);
    SKN_REQUIRE(ctx, k % be == 0, SKN_ERR_SHAPE,
                "Quantized tensor row size (%d) is not a multiple of block size (%d)", k, be);
    if (n == 0) return SKN_OK;
    SKN_REQUIRE(ctx, y_dev != nullptr, SKN_ERR_ARG, "skn_matvec_q: y is null");
    if (k == 0) return skn_memset(ctx, y_dev, 0, (size_t)n * sizeof(float));
    SKN_REQUIRE(ctx, w_dev && x_dev, SKN_ERR_ARG, "skn_matvec_q: null pointer");
    SKN_REQUIRE(ctx, ((uintptr_t)x_dev & 15) == 0, SKN_ERR_ARG, "skn_matvec_q: x must be 16-byte aligned");
    SKN_REQUIRE(ctx, ((uintptr_t)w_dev & (ggml_type == SKN_TYPE_Q4_K ? 15 : 1)) == 0, SKN_ERR_ARG,
                "skn_matvec_q: weight pointer is misaligned for its block type");
    const uint8_t* w = (const uint8_t*)w_dev;
    const int nb = k / be;
    if (ggml_type == SKN_TYPE_Q4_K) {
        const int steps = (nb + 7) / 8;
        const int waves = 16;
        switch (steps) {
            case 1: return launch_q4k<1>(ctx, w, n, nb, x_dev, y_dev, waves);
            case 2: return launch_q4k<2>(ctx, w, n, nb, x_dev, y_dev, waves);
            case 3: return launch_q4k<3>(ctx, w, n, nb, x_dev, y_dev, waves);
            case 4: return launch_q4k<4>(ctx, w, n, nb, x_dev, y_dev, waves);
            case 6: return launch_q4k<6>(ctx, w, n, nb, x_dev, y_dev, waves);
            case 7: return launch_q4k<7>(ctx, w, n, nb, x_dev, y_dev, waves);
            default: return launch_q4k<0>(ctx, w, n, nb, x_dev, y_dev, waves);
        }
    }
    dim3 grid((unsigned)((n + 3) / 4)), block(256);
    if (ggml_type == SKN_TYPE_Q8_0)
        skn_launch(ctx, matvec_q8_0_kernel, grid, block, 0, w, x_dev, y_dev, n, nb);
    else
        skn_launch(ctx, matvec_q6_k_kernel, grid, block, 0, w, x_dev, y_dev, n, nb);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}
