// Batched quantized GEMM  C[m,n] = sum_k A[m,k] * deq(W)[n,k]  (A bf16 [m,k], W GGUF blocks [n,k], C fp32 [m,n])
// on the matrix cores (v_mfma_f32_32x32x16_f16, fp32 accumulation).
//
// The tolerance asked of this op (1e-3 of max(|c|, 1e-3 * max|c|)) needs about 20 bits of every weight: a
// dequantized weight rounded to one fp16 / bf16 operand (11 / 8 bits) would miss it on outputs near zero.
// Both paths below therefore feed the MFMA with operands that are exact or exact to 2^-22:
//
//   * Activations: bf16 -> fp16 is exact for every value whose magnitude is within fp16 range; a row whose
//     largest magnitude exceeds 2^14 is scaled down by a power of two first and the scale undone in the
//     epilogue (prep_a_kernel).  Products and sums are fp32 inside the MFMA.
//   * Weights, general path (Q8_0, Q6_K): W is dequantized once into a workspace as an fp16 pair
//     hi = f16(w), lo = f16(w - hi) (w_hi + w_lo = w to 2^-22 relative) and each k-step issues two MFMAs.
//   * Weights, Q4_K path: see gemm_q4k_kernel -- the 4-bit quants times their 6-bit sub-block scale are
//     integers below 2^10, exact in fp16, so one MFMA per k-step suffices and the f16 superblock scale d is
//     applied to the fp32 partial sum of each superblock.
#include "common.h"

namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kBM = 128;  // workgroup tile rows (activations)
constexpr int kBN = 64;   // workgroup tile columns (weight rows)
constexpr int kKC = 64;   // k elements staged in LDS per iteration
constexpr int kRow = kKC + 8;  // LDS row pitch in halves: 144 bytes keeps 128-bit reads of 16 rows conflict-free

// ---- activation preparation: bf16 [m,k] -> fp16 [m,k] with a per-row power-of-two scale -------------------
// One workgroup per row.  Also emits, for the Q4_K path, the per-32-element sums of the fp16 row as an fp16
// pair (hi, lo), and can write the row in the element order the Q4_K kernel consumes (PERMUTE).
template <bool Q4K>
__global__ __launch_bounds__(256) void prep_a_kernel(const uint16_t* __restrict__ a, _Float16* __restrict__ a16,
                                                     float* __restrict__ inv_scale, _Float16* __restrict__ sum_hi,
                                                     _Float16* __restrict__ sum_lo, int k) {
    __shared__ float red[4];
    const int m = blockIdx.x;
    const uint16_t* ar = a + (size_t)m * k;
    float mx = 0.f;
    for (int i = threadIdx.x; i < k; i += 256) {
        const float v = fabsf(__uint_as_float((uint32_t)ar[i] << 16));
        if (v == v && v < INFINITY) mx = fmaxf(mx, v);
    }
    mx = wave_max(mx);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    // scale = 2^-e with the smallest e >= 0 such that mx * scale <= 2^14
    int e = 0;
    if (mx > 16384.f) e = (int)((__float_as_uint(mx) >> 23) & 0xFF) - 127 - 14 + 1;
    const float scale = __uint_as_float((uint32_t)(127 - e) << 23);
    if (threadIdx.x == 0) inv_scale[m] = __uint_as_float((uint32_t)(127 + e) << 23);
    _Float16* out = a16 + (size_t)m * k;
    if (!Q4K) {
        for (int i = threadIdx.x; i < k; i += 256) out[i] = (_Float16)(__uint_as_float((uint32_t)ar[i] << 16) * scale);
    } else {
        // one thread per 32-element sub-block: its sum, and the permuted store
        const int nsub = k >> 5;
        for (int s = threadIdx.x; s < nsub; s += 256) {
            float sum = 0.f;
            const int chunk = s >> 1, upper = s & 1;  // 64-element chunk, lower / upper 32 elements
            for (int i = 0; i < 32; i++) {
                const _Float16 h = (_Float16)(__uint_as_float((uint32_t)ar[32 * s + i] << 16) * scale);
                sum += (float)h;
                // element 32*upper + 4*dw + b of the chunk (dw = dword of nibble bytes, b = byte in it) goes to
                // position dw*8 + {0,4,1,5}[b] + 2*upper: the order the nibble masks of the Q4_K kernel produce
                const int dw = i >> 2, b = i & 3;
                const int pos = dw * 8 + ((b & 1) << 2) + (b >> 1) + 2 * upper;
                out[64 * chunk + pos] = h;
            }
            const _Float16 hi = (_Float16)sum;
            sum_hi[(size_t)m * nsub + s] = hi;
            sum_lo[(size_t)m * nsub + s] = (_Float16)(sum - (float)hi);
        }
    }
}

// fp32 [n] -> fp16 pair (hi, lo)
__global__ void split_hilo_kernel(const float* __restrict__ w, _Float16* __restrict__ hi, _Float16* __restrict__ lo,
                                  int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const float v = w[i];
        const _Float16 h = (_Float16)v;
        hi[i] = h;
        lo[i] = (_Float16)(v - (float)h);
    }
}

// C tile store: acc register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32 of the 32x32 tile
__device__ __forceinline__ void store_tile(const float16_t& acc, float* __restrict__ c, int ldc, int row0, int col0,
                                           int m, int n, const float* __restrict__ inv_scale, int lane) {
    const int col = col0 + (lane & 31);
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int row = row0 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (row < m && col < n) c[(size_t)row * ldc + col] = acc[r] * inv_scale[row];
    }
}

// ---- general path: dense fp16 activations x (hi + lo) fp16 weights ----------------------------------------
// Workgroup 256 threads = 2 x 2 wavefronts; workgroup tile 128 x 64; wavefront tile 64 x 32 = two 32x32 MFMA
// tiles sharing one pair of weight fragments.  A, W_hi, W_lo tiles of 64 k go through LDS; the next tiles are
// fetched into registers while the current ones are consumed.
__global__ __launch_bounds__(256) void gemm_dense_hilo_kernel(const _Float16* __restrict__ a16,
                                                              const _Float16* __restrict__ whi,
                                                              const _Float16* __restrict__ wlo,
                                                              const float* __restrict__ inv_scale, float* __restrict__ c,
                                                              int m, int n, int k) {
    __shared__ __align__(16) _Float16 sa[kBM * kRow];
    __shared__ __align__(16) _Float16 sh[kBN * kRow];
    __shared__ __align__(16) _Float16 sl[kBN * kRow];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * kBM, n0 = blockIdx.x * kBN;

    // global -> register staging: A tile 128 rows x 8 chunks of 16 B = 1024 chunks (4 per thread),
    // W tiles 64 rows x 8 chunks = 512 chunks each (2 per thread)
    uint4 ra0, ra1, ra2, ra3, rh0, rh1, rl0, rl1;
    const int srow = tid >> 3, sch = (tid & 7) * 8;  // this thread's row (+32 per slot) and column of the tiles
    const _Float16* ga0 = a16 + (size_t)min(m0 + srow, m - 1) * k + sch;
    const _Float16* ga1 = a16 + (size_t)min(m0 + srow + 32, m - 1) * k + sch;
    const _Float16* ga2 = a16 + (size_t)min(m0 + srow + 64, m - 1) * k + sch;
    const _Float16* ga3 = a16 + (size_t)min(m0 + srow + 96, m - 1) * k + sch;
    const size_t gw0 = (size_t)min(n0 + srow, n - 1) * k + sch;
    const size_t gw1 = (size_t)min(n0 + srow + 32, n - 1) * k + sch;
#define SKN_FETCH(k0)                                              \
    do {                                                           \
        ra0 = *reinterpret_cast<const uint4*>(ga0 + (k0));         \
        ra1 = *reinterpret_cast<const uint4*>(ga1 + (k0));         \
        ra2 = *reinterpret_cast<const uint4*>(ga2 + (k0));         \
        ra3 = *reinterpret_cast<const uint4*>(ga3 + (k0));         \
        rh0 = *reinterpret_cast<const uint4*>(whi + gw0 + (k0));   \
        rh1 = *reinterpret_cast<const uint4*>(whi + gw1 + (k0));   \
        rl0 = *reinterpret_cast<const uint4*>(wlo + gw0 + (k0));   \
        rl1 = *reinterpret_cast<const uint4*>(wlo + gw1 + (k0));   \
    } while (0)
#define SKN_STASH()                                                                  \
    do {                                                                             \
        *reinterpret_cast<uint4*>(sa + srow * kRow + sch) = ra0;                     \
        *reinterpret_cast<uint4*>(sa + (srow + 32) * kRow + sch) = ra1;              \
        *reinterpret_cast<uint4*>(sa + (srow + 64) * kRow + sch) = ra2;              \
        *reinterpret_cast<uint4*>(sa + (srow + 96) * kRow + sch) = ra3;              \
        *reinterpret_cast<uint4*>(sh + srow * kRow + sch) = rh0;                     \
        *reinterpret_cast<uint4*>(sh + (srow + 32) * kRow + sch) = rh1;              \
        *reinterpret_cast<uint4*>(sl + srow * kRow + sch) = rl0;                     \
        *reinterpret_cast<uint4*>(sl + (srow + 32) * kRow + sch) = rl1;              \
    } while (0)

    float16_t acc0, acc1;
#pragma unroll
    for (int r = 0; r < 16; r++) acc0[r] = acc1[r] = 0.f;

    SKN_FETCH(0);
    for (int k0 = 0; k0 < k; k0 += kKC) {
        __syncthreads();  // everyone is done reading the previous tiles
        SKN_STASH();
        __syncthreads();
        if (k0 + kKC < k) SKN_FETCH(k0 + kKC);
        const _Float16* pa0 = sa + (wm * 64 + (lane & 31)) * kRow + (lane >> 5) * 8;
        const _Float16* pa1 = pa0 + 32 * kRow;
        const _Float16* ph = sh + (wn * 32 + (lane & 31)) * kRow + (lane >> 5) * 8;
        const _Float16* pl = sl + (wn * 32 + (lane & 31)) * kRow + (lane >> 5) * 8;
#pragma unroll
        for (int t = 0; t < kKC / 16; t++) {
            const half8_t fa0 = *reinterpret_cast<const half8_t*>(pa0 + 16 * t);
            const half8_t fa1 = *reinterpret_cast<const half8_t*>(pa1 + 16 * t);
            const half8_t fh = *reinterpret_cast<const half8_t*>(ph + 16 * t);
            const half8_t fl = *reinterpret_cast<const half8_t*>(pl + 16 * t);
            acc0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa0, fh, acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa1, fh, acc1, 0, 0, 0);
            acc0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa0, fl, acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa1, fl, acc1, 0, 0, 0);
        }
    }
    store_tile(acc0, c, n, m0 + wm * 64, n0 + wn * 32, m, n, inv_scale, lane);
    store_tile(acc1, c, n, m0 + wm * 64 + 32, n0 + wn * 32, m, n, inv_scale, lane);
#undef SKN_FETCH
#undef SKN_STASH
}

// grows the context's GEMM workspace; the pointer stays valid until the next growth
int gemm_workspace(skn_ctx* ctx, size_t bytes, uint8_t** out) {
    if (bytes > ctx->gemm_ws_bytes) {
        SKN_HIP(ctx, hipStreamSynchronize(ctx->stream));
        if (ctx->gemm_ws) SKN_HIP(ctx, hipFree(ctx->gemm_ws));
        ctx->gemm_ws = nullptr;
        ctx->gemm_ws_bytes = 0;
        hipError_t e = hipMalloc(&ctx->gemm_ws, bytes);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return skn_fail(ctx, SKN_ERR_OOM, "skn_gemm_q: %zu bytes of workspace: %s", bytes, hipGetErrorString(e));
        }
        ctx->gemm_ws_bytes = bytes;
    }
    *out = (uint8_t*)ctx->gemm_ws;
    return SKN_OK;
}

inline size_t align_up(size_t v) { return (v + 255) & ~(size_t)255; }

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
    SKN_REQUIRE(ctx, k % kKC == 0, SKN_ERR_SHAPE, "skn_gemm_q: k (%d) must be a multiple of %d", k, kKC);

    // workspace: fp16 activations + row scales, then (general path) fp32 weights and their fp16 pair
    const size_t a16_bytes = align_up((size_t)m * k * 2), sc_bytes = align_up((size_t)m * 4);
    const size_t wf_bytes = align_up((size_t)n * k * 4), wh_bytes = align_up((size_t)n * k * 2);
    uint8_t* ws;
    int rc = gemm_workspace(ctx, a16_bytes + sc_bytes + wf_bytes + 2 * wh_bytes, &ws);
    if (rc != SKN_OK) return rc;
    _Float16* a16 = (_Float16*)ws;
    float* inv_scale = (float*)(ws + a16_bytes);
    float* wf = (float*)(ws + a16_bytes + sc_bytes);
    _Float16* whi = (_Float16*)(ws + a16_bytes + sc_bytes + wf_bytes);
    _Float16* wlo = (_Float16*)(ws + a16_bytes + sc_bytes + wf_bytes + wh_bytes);

    skn_launch(ctx, prep_a_kernel<false>, dim3(m), dim3(256), 0, a_bf16_dev, a16, inv_scale, (_Float16*)nullptr,
               (_Float16*)nullptr, k);
    SKN_LAUNCH_CHECK(ctx);
    rc = skn_dequant(ctx, ggml_type, w_dev, (int64_t)n * k, wf);
    if (rc != SKN_OK) return rc;
    const int64_t total = (int64_t)n * k;
    skn_launch(ctx, split_hilo_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (const float*)wf, whi, wlo,
               total);
    SKN_LAUNCH_CHECK(ctx);
    dim3 grid((n + kBN - 1) / kBN, (m + kBM - 1) / kBM);
    skn_launch(ctx, gemm_dense_hilo_kernel, grid, dim3(256), 0, (const _Float16*)a16, (const _Float16*)whi,
               (const _Float16*)wlo, (const float*)inv_scale, c_dev, m, n, k);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}
