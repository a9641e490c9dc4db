// Machine measurements the design leans on, runnable from the library (bench.py --mode machine): how far vector
// instructions hide behind matrix instructions on a SIMD, and how fast 1 KiB operand fragments arrive in a compute
// unit's registers.  Test hooks: no part of the inference path.
#include "common.h"

namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Four v_mfma_f32_32x32x16_f16 into four accumulators per iteration, each followed by NV v_and_b32 on eight other
// registers (independent of the matrix instructions and, eight apart, of each other).
template <int NV>
__global__ __launch_bounds__(512) void mfma_valu_kernel(float* out, int iters, unsigned seed) {
    half8_t a, b;
    for (int i = 0; i < 8; i++) {
        a[i] = (_Float16)(float)((threadIdx.x + i) & 3);
        b[i] = (_Float16)(float)((threadIdx.x * 3 + i) & 3);
    }
    float16_t c[4];
    for (int j = 0; j < 4; j++)
        for (int i = 0; i < 16; i++) c[j][i] = 0.f;
    unsigned v[8];
    for (int i = 0; i < 8; i++) v[i] = seed + threadIdx.x * (i + 1);
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            c[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c[j], 0, 0, 0);
#pragma unroll
            for (int q = 0; q < NV; q++) asm volatile("v_and_b32 %0, 0x0fff0fff, %0" : "+v"(v[(j * NV + q) & 7]));
        }
    }
    float s = 0.f;
    for (int j = 0; j < 4; j++)
        for (int i = 0; i < 16; i++) s += c[j][i];
    unsigned u = 0;
    for (int i = 0; i < 8; i++) u ^= v[i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s + (float)u;
}

// Every wavefront streams `steps` fragments of 1 KiB (one 16-byte load per lane) through a ring of eight registers
// sets; SHARE wavefronts of a workgroup read the same stream.
template <int SHARE>
__global__ __launch_bounds__(512) void fragment_kernel(const u32x4* __restrict__ a, unsigned* out, int steps, int streams) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int stream = (blockIdx.x * (8 / SHARE) + wave / SHARE) % streams;
    const u32x4* p = a + (size_t)stream * steps * 64 + lane;
    u32x4 acc = {0, 0, 0, 0};
    u32x4 r[8];
#pragma unroll
    for (int i = 0; i < 8; i++) r[i] = p[i * 64];
    for (int s = 8; s + 8 <= steps; s += 8) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            acc ^= r[i];
            r[i] = p[(s + i) * 64];
        }
    }
#pragma unroll
    for (int i = 0; i < 8; i++) acc ^= r[i];
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x1234567u) out[0] = 1;
}

template <typename F>
int time_launches(skn_ctx* ctx, int reps, F launch, double* us_per_launch) {
    hipEvent_t e0, e1;
    SKN_HIP(ctx, hipEventCreate(&e0));
    SKN_HIP(ctx, hipEventCreate(&e1));
    for (int i = 0; i < 3; i++) launch();
    SKN_HIP(ctx, hipEventRecord(e0, ctx->stream));
    for (int i = 0; i < reps; i++) launch();
    SKN_HIP(ctx, hipEventRecord(e1, ctx->stream));
    SKN_HIP(ctx, hipEventSynchronize(e1));
    float ms = 0.f;
    SKN_HIP(ctx, hipEventElapsedTime(&ms, e0, e1));
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    SKN_LAUNCH_CHECK(ctx);
    *us_per_launch = (double)ms * 1e3 / reps;
    return SKN_OK;
}

}  // namespace

// ns per matrix instruction and SIMD with `valu_per_mfma` (0, 2, 4, 6, 7, 8 or 12) independent vector instructions behind
// each, at one or two wavefronts per SIMD.  scratch_dev: 512 KiB of device memory.
extern "C" int skn_test_mfma_valu_overlap(skn_ctx* ctx, int waves_per_simd, int valu_per_mfma, float* scratch_dev, double* ns_out) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_test_mfma_valu_overlap: ctx is null");
    SKN_REQUIRE(ctx, scratch_dev && ns_out && (waves_per_simd == 1 || waves_per_simd == 2), SKN_ERR_ARG,
                "skn_test_mfma_valu_overlap: bad arguments");
    const int iters = 4000, block = 256 * waves_per_simd, grid = ctx->compute_units;
    SKN_REQUIRE(ctx, grid * block * sizeof(float) <= 512 * 1024, SKN_ERR_SHAPE, "skn_test_mfma_valu_overlap: scratch too small");
    double us = 0.0;
    int rc;
#define SKN_CASE(NV)                                                                                                      \
    case NV:                                                                                                              \
        rc = time_launches(ctx, 5, [&] { skn_launch(ctx, mfma_valu_kernel<NV>, dim3(grid), dim3(block), 0, scratch_dev, iters, 1u); }, &us); \
        break;
    switch (valu_per_mfma) {
        SKN_CASE(0) SKN_CASE(2) SKN_CASE(4) SKN_CASE(6) SKN_CASE(7) SKN_CASE(8) SKN_CASE(12)
        default: return skn_fail(ctx, SKN_ERR_ARG, "skn_test_mfma_valu_overlap: %d vector instructions per matrix instruction is not built", valu_per_mfma);
    }
#undef SKN_CASE
    if (rc != SKN_OK) return rc;
    // per launch and SIMD: iters * 4 matrix instructions per wavefront, waves_per_simd wavefronts
    *ns_out = us * 1e3 / ((double)iters * 4 * waves_per_simd);
    return SKN_OK;
}

// GB/s per compute unit into the registers when `share` (1, 2, 4 or 8) wavefronts of a workgroup read the same
// fragments.  data_dev: data_mib MiB of device memory (any content), a multiple of 1 MiB; each wavefront reads 1 MiB.
extern "C" int skn_test_fragment_delivery(skn_ctx* ctx, int share, const void* data_dev, int data_mib, unsigned* flag_dev, double* gbs_out) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_test_fragment_delivery: ctx is null");
    SKN_REQUIRE(ctx, data_dev && flag_dev && gbs_out && data_mib >= 1 && ((uintptr_t)data_dev & 15) == 0, SKN_ERR_ARG,
                "skn_test_fragment_delivery: bad arguments");
    const int steps = 1024, grid = ctx->compute_units;
    const u32x4* a = (const u32x4*)data_dev;
    double us = 0.0;
    int rc;
    switch (share) {
        case 1: rc = time_launches(ctx, 10, [&] { skn_launch(ctx, fragment_kernel<1>, dim3(grid), dim3(512), 0, a, flag_dev, steps, data_mib); }, &us); break;
        case 2: rc = time_launches(ctx, 10, [&] { skn_launch(ctx, fragment_kernel<2>, dim3(grid), dim3(512), 0, a, flag_dev, steps, data_mib); }, &us); break;
        case 4: rc = time_launches(ctx, 10, [&] { skn_launch(ctx, fragment_kernel<4>, dim3(grid), dim3(512), 0, a, flag_dev, steps, data_mib); }, &us); break;
        case 8: rc = time_launches(ctx, 10, [&] { skn_launch(ctx, fragment_kernel<8>, dim3(grid), dim3(512), 0, a, flag_dev, steps, data_mib); }, &us); break;
        default: return skn_fail(ctx, SKN_ERR_ARG, "skn_test_fragment_delivery: share must be 1, 2, 4 or 8");
    }
    if (rc != SKN_OK) return rc;
    *gbs_out = 8.0 * steps * 1024.0 / us / 1e3;  // eight wavefronts x steps KiB per compute unit and launch
    return SKN_OK;
}
