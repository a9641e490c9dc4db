// Batched quantized GEMM  C[m,n] = sum_k A[m,k] * deq(W)[n,k]  (A bf16, C fp32).
// Provisional form: one matvec per activation row on fp32-converted activations.
#include "common.h"

namespace {
__global__ void bf16_to_f32_kernel(const uint16_t* __restrict__ a, float* __restrict__ out, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = __uint_as_float((uint32_t)a[i] << 16);
}
}  // namespace

extern "C" int skn_gemm_q(skn_ctx* ctx, int ggml_type, const void* w_dev, int n, int k, const uint16_t* a_bf16_dev,
                          int m, float* c_dev) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_gemm_q: ctx is null");
    SKN_REQUIRE(ctx, skn_is_quant(ggml_type), SKN_ERR_TYPE, "skn_gemm_q: ggml type %d is not supported", ggml_type);
    SKN_REQUIRE(ctx, n >= 0 && k >= 0 && m >= 0, SKN_ERR_ARG, "skn_gemm_q: negative shape");
    int be, bb;
    skn_type_block(ggml_type, &be, &bb);
    SKN_REQUIRE(ctx, k % be == 0, SKN_ERR_SHAPE, "Quantized tensor row size (%d) is not a multiple of block size (%d)", k,
                be);
    if (n == 0 || m == 0) return SKN_OK;
    SKN_REQUIRE(ctx, c_dev != nullptr, SKN_ERR_ARG, "skn_gemm_q: c is null");
    if (k == 0) return skn_memset(ctx, c_dev, 0, (size_t)m * n * sizeof(float));
    SKN_REQUIRE(ctx, w_dev && a_bf16_dev, SKN_ERR_ARG, "skn_gemm_q: null pointer");
    float* af = nullptr;
    hipError_t e = hipMalloc((void**)&af, (size_t)m * k * sizeof(float));
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return skn_fail(ctx, SKN_ERR_OOM, "skn_gemm_q: workspace: %s", hipGetErrorString(e));
    }
    const int64_t total = (int64_t)m * k;
    skn_launch(ctx, bf16_to_f32_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, a_bf16_dev,
                       af, total);
    int rc = SKN_OK;
    for (int r = 0; r < m && rc == SKN_OK; r++)
        rc = skn_matvec_q(ctx, ggml_type, w_dev, n, k, af + (size_t)r * k, c_dev + (size_t)r * n);
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipFree(af);
    return rc;
}
