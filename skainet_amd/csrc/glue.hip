// Decoder glue in fp32: RMSNorm, rotary embedding, SwiGLU, residual add, argmax, fp32 -> fp16 / bf16.
// All are a few KB to a few MB per call and HBM / launch bound; none of them is on the weight stream.
#include "common.h"

namespace {

__global__ __launch_bounds__(256) void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                      float* __restrict__ y, int n, float eps) {
    __shared__ float red[4];
    const float* xr = x + (size_t)blockIdx.x * n;
    float* yr = y + (size_t)blockIdx.x * n;
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += 256) ss = fmaf(xr[i], xr[i], ss);
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float total = (red[0] + red[1]) + (red[2] + red[3]);
    const float r = 1.0f / sqrtf(total / (float)n + eps);
    for (int i = threadIdx.x; i < n; i += 256) yr[i] = xr[i] * r * w[i];
}

// one thread per (row, head, pair)
__global__ void rope_kernel(float* __restrict__ x, int rows, int n_head, int head_dim, int pos0, double log2_base) {
    const int half = head_dim >> 1;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t total = (int64_t)rows * n_head * half;
    if (idx >= total) return;
    const int i = (int)(idx % half);
    const int64_t rh = idx / half;
    const int row = (int)(rh / n_head);
    float sn, cs;
    skn_rope_sincos(pos0 + row, 2 * i, head_dim, log2_base, &sn, &cs);
    float* p = x + rh * head_dim + 2 * i;
    const float a = p[0], b = p[1];
    p[0] = a * cs - b * sn;
    p[1] = a * sn + b * cs;
}

__global__ void swiglu_kernel(const float* __restrict__ g, const float* __restrict__ u, float* __restrict__ out,
                              int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const float a = g[i];
        out[i] = a / (1.0f + expf(-a)) * u[i];
    }
}

__global__ void relu_kernel(const float* __restrict__ x, float* __restrict__ out, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const float v = x[i];
        out[i] = v > 0.f ? v : 0.f;  // (a NaN becomes 0, as `if (elem > 0) elem else 0.0` makes it)
    }
}

__global__ void add_kernel(float* __restrict__ y, const float* __restrict__ x, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] += x[i];
}

// single workgroup of 1024 threads; first index of the maximum
__global__ __launch_bounds__(1024) void argmax_kernel(const float* __restrict__ x, int n, int32_t* __restrict__ out) {
    __shared__ float bv[16];
    __shared__ int bi[16];
    float best = -INFINITY;
    int besti = 0x7FFFFFFF;
    for (int i = threadIdx.x; i < n; i += 1024) {
        const float v = x[i];
        if (v > best || (v == best && i < besti)) {
            best = v;
            besti = i;
        }
    }
    for (int off = 32; off >= 1; off >>= 1) {
        const float ov = __shfl_xor(best, off, 64);
        const int oi = __shfl_xor(besti, off, 64);
        if (ov > best || (ov == best && oi < besti)) {
            best = ov;
            besti = oi;
        }
    }
    if ((threadIdx.x & 63) == 0) {
        bv[threadIdx.x >> 6] = best;
        bi[threadIdx.x >> 6] = besti;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; w++)
            if (bv[w] > best || (bv[w] == best && bi[w] < besti)) {
                best = bv[w];
                besti = bi[w];
            }
        *out = besti == 0x7FFFFFFF ? 0 : besti;
    }
}

__global__ void f32_to_f16_kernel(const float* __restrict__ x, uint16_t* __restrict__ out, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = __half_as_ushort(__float2half_rn(x[i]));
}

__global__ void f32_to_bf16_kernel(const float* __restrict__ x, uint16_t* __restrict__ out, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        uint32_t u = __float_as_uint(x[i]);
        if ((u & 0x7FFFFFFFu) > 0x7F800000u) {
            out[i] = (uint16_t)((u >> 16) | 0x40u);
        } else {
            u += 0x7FFFu + ((u >> 16) & 1u);
            out[i] = (uint16_t)(u >> 16);
        }
    }
}

inline unsigned blocks_for(int64_t n, int per) { return (unsigned)((n + per - 1) / per); }

}  // namespace

extern "C" {

int skn_rmsnorm(skn_ctx* ctx, const float* x_dev, const float* w_dev, int rows, int n, float eps, float* y_dev) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_rmsnorm: ctx is null");
    SKN_REQUIRE(ctx, rows >= 0 && n > 0, SKN_ERR_ARG, "skn_rmsnorm: bad shape");
    if (rows == 0) return SKN_OK;
    SKN_REQUIRE(ctx, x_dev && w_dev && y_dev, SKN_ERR_ARG, "skn_rmsnorm: null pointer");
    skn_launch(ctx, rmsnorm_kernel, dim3(rows), dim3(256), 0, x_dev, w_dev, y_dev, n, eps);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

int skn_rope(skn_ctx* ctx, float* x_dev, int rows, int n_head, int head_dim, int pos0, float base) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_rope: ctx is null");
    SKN_REQUIRE(ctx, rows >= 0 && n_head > 0 && head_dim > 0 && head_dim % 2 == 0 && base > 0.f, SKN_ERR_ARG,
                "skn_rope: bad shape");
    if (rows == 0) return SKN_OK;
    SKN_REQUIRE(ctx, x_dev != nullptr, SKN_ERR_ARG, "skn_rope: null pointer");
    const int64_t total = (int64_t)rows * n_head * (head_dim / 2);
    skn_launch(ctx, rope_kernel, dim3(blocks_for(total, 256)), dim3(256), 0, x_dev, rows, n_head,
                       head_dim, pos0, log2((double)base));
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

int skn_swiglu(skn_ctx* ctx, const float* gate_dev, const float* up_dev, int64_t n, float* out_dev) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_swiglu: ctx is null");
    SKN_REQUIRE(ctx, n >= 0, SKN_ERR_ARG, "skn_swiglu: negative size");
    if (n == 0) return SKN_OK;
    SKN_REQUIRE(ctx, gate_dev && up_dev && out_dev, SKN_ERR_ARG, "skn_swiglu: null pointer");
    skn_launch(ctx, swiglu_kernel, dim3(blocks_for(n, 256)), dim3(256), 0, gate_dev, up_dev, out_dev, n);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

int skn_relu(skn_ctx* ctx, const float* x_dev, int64_t n, float* out_dev) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_relu: ctx is null");
    SKN_REQUIRE(ctx, n >= 0, SKN_ERR_ARG, "skn_relu: negative size");
    if (n == 0) return SKN_OK;
    SKN_REQUIRE(ctx, x_dev && out_dev, SKN_ERR_ARG, "skn_relu: null pointer");
    skn_launch(ctx, relu_kernel, dim3(blocks_for(n, 256)), dim3(256), 0, x_dev, out_dev, n);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

int skn_add_inplace(skn_ctx* ctx, float* y_dev, const float* x_dev, int64_t n) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_add_inplace: ctx is null");
    SKN_REQUIRE(ctx, n >= 0, SKN_ERR_ARG, "skn_add_inplace: negative size");
    if (n == 0) return SKN_OK;
    SKN_REQUIRE(ctx, y_dev && x_dev, SKN_ERR_ARG, "skn_add_inplace: null pointer");
    skn_launch(ctx, add_kernel, dim3(blocks_for(n, 256)), dim3(256), 0, y_dev, x_dev, n);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

int skn_argmax(skn_ctx* ctx, const float* x_dev, int n, int32_t* index_dev) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_argmax: ctx is null");
    SKN_REQUIRE(ctx, n > 0, SKN_ERR_ARG, "skn_argmax: empty input");
    SKN_REQUIRE(ctx, x_dev && index_dev, SKN_ERR_ARG, "skn_argmax: null pointer");
    skn_launch(ctx, argmax_kernel, dim3(1), dim3(1024), 0, x_dev, n, index_dev);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

int skn_f32_to_f16(skn_ctx* ctx, const float* x_dev, int64_t n, uint16_t* out_dev) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_f32_to_f16: ctx is null");
    SKN_REQUIRE(ctx, n >= 0, SKN_ERR_ARG, "skn_f32_to_f16: negative size");
    if (n == 0) return SKN_OK;
    SKN_REQUIRE(ctx, x_dev && out_dev, SKN_ERR_ARG, "skn_f32_to_f16: null pointer");
    skn_launch(ctx, f32_to_f16_kernel, dim3(blocks_for(n, 256)), dim3(256), 0, x_dev, out_dev, n);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

int skn_f32_to_bf16(skn_ctx* ctx, const float* x_dev, int64_t n, uint16_t* out_dev) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_f32_to_bf16: ctx is null");
    SKN_REQUIRE(ctx, n >= 0, SKN_ERR_ARG, "skn_f32_to_bf16: negative size");
    if (n == 0) return SKN_OK;
    SKN_REQUIRE(ctx, x_dev && out_dev, SKN_ERR_ARG, "skn_f32_to_bf16: null pointer");
    skn_launch(ctx, f32_to_bf16_kernel, dim3(blocks_for(n, 256)), dim3(256), 0, x_dev, out_dev, n);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

}  // extern "C"
