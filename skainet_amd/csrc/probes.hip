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

// A model of the Q4_K GEMM's inner loop (gemm.hip, gemm_q4k_frag_kernel<2, 2>: two wavefronts per SIMD, a 64 x 64
// register tile per wavefront, sixteen k-steps of four matrix instructions per superblock) whose parts can be left
// out, to see what each costs next to the matrix instructions.  PARTS, bit by bit: 1 the nibble decode that feeds the
// weight operand (one step ahead), 2 nibbles read from LDS and the per-chunk scale unpack, 4 activation fragments from
// memory through a ring of eight steps, 8 the per-superblock header unpack (scales, mins, units), 16 the accumulator
// rescale, 32 the "- dmin * m" term (two more matrix instructions per tile and the hi | lo split of its operand).
// The arithmetic is that of the kernel on arbitrary bits; the results mean nothing.
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
template <int PARTS>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void q4k_loop_kernel(const u32x4* __restrict__ afrag, uint32_t a_bytes, float* out, int superblocks, unsigned seed) {
    constexpr int MT = 2, kPitch = 592;
    __shared__ __align__(16) uint8_t lds[64 * kPitch];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = lane >> 5, r = lane & 31;
    for (int i = tid; i < 64 * kPitch / 4; i += 512) ((uint32_t*)lds)[i] = seed * 2654435761u + i * 40503u;
    __syncthreads();
    const __amdgpu_buffer_rsrc_t arsrc = __builtin_amdgcn_make_buffer_rsrc((void*)afrag, 0, (int)a_bytes, 0x00020000);
    // each wavefront streams 1 MiB of its own (one of 64 such regions), again and again
    const uint32_t wbase = (uint32_t)((blockIdx.x * 8 + wave) % 64) * (uint32_t)(a_bytes / 64);
    u32x4 a[8][MT];
    auto afetch = [&](int step, int slot) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < MT; i++)
            a[slot][i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(arsrc, lane * 16, (int)(wbase + (uint32_t)((step * MT + i) & 1023) * 1024u), 0));
    };
    float16_t acc[MT][2];
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int x = 0; x < 16; x++) acc[i][j][x] = 0.f;
#pragma unroll
    for (int s = 0; s < 8; s++) {
        if (PARTS & 4) {
            afetch(s, s);
        } else {
#pragma unroll
            for (int i = 0; i < MT; i++) a[s][i] = u32x4{0x3c003c00u + (unsigned)lane, 0x3c003c00u, 0x38003800u, 0x3c003c00u};
        }
    }
    const uint8_t* wl = lds + r * kPitch + (wave & 3) * 144;
    constexpr int kTile = 32 * kPitch;
    u32x4 q[2], qn[2];
    half2_t mul_lo[2], mul_hi[2];
    half8_t fb[2], fbn[2];
    uint32_t sc4[2][2] = {{seed & 0x3F3F3F3Fu, (seed >> 1) & 0x3F3F3F3Fu}, {(seed >> 2) & 0x3F3F3F3Fu, (seed >> 3) & 0x3F3F3F3Fu}};
    uint32_t mn4[2][2] = {{1, 2}, {3, 4}};
    float sc_unit[2] = {1.0f / 1024, 1.0f / 1024}, cs[2] = {1.f, 1.f}, min_unit[2] = {0.f, 0.f};
    auto byte_f = [](uint32_t word, int b) { return (float)((word >> (8 * b)) & 0xFFu); };
    auto load_q = [&](int cc, u32x4* dst) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            if (PARTS & 2) {
                dst[j] = *reinterpret_cast<const u32x4*>(wl + j * kTile + 16 + 32 * cc + 16 * h);
            } else {
                dst[j] = u32x4{seed + lane, seed * 3 + lane, seed * 5 + lane, seed * 7 + lane};
                asm volatile("" : "+v"(dst[j]));  // (opaque: not hoisted out of the loop)
            }
        }
    };
    auto scales = [&](int cc) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const float fl = byte_f(sc4[j][cc >> 1], 2 * (cc & 1)) * sc_unit[j];
            const float fh = byte_f(sc4[j][cc >> 1], 2 * (cc & 1) + 1) * (sc_unit[j] * 0.0625f);
            mul_lo[j] = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_pkrtz(fl, fl));
            mul_hi[j] = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_pkrtz(fh, fh));
        }
    };
    auto decode = [&](int s, half8_t* dst) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const uint32_t qq = q[j][s], q8 = qq >> 8;
            const uint32_t l02 = qq & 0x000F000Fu, h02 = qq & 0x00F000F0u;
            const uint32_t l13 = q8 & 0x000F000Fu, h13 = q8 & 0x00F000F0u;
            u32x4 o;
            o.x = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, l02) * mul_lo[j]);
            o.y = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, h02) * mul_hi[j]);
            o.z = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, l13) * mul_lo[j]);
            o.w = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, h13) * mul_hi[j]);
            dst[j] = __builtin_bit_cast(half8_t, o);
        }
    };
    constexpr bool DEC = (PARTS & 1) != 0;
    for (int sb = 0; sb < superblocks; sb++) {
        if (PARTS & 8) {
            u32x4 hd[2];
#pragma unroll
            for (int j = 0; j < 2; j++) hd[j] = *reinterpret_cast<const u32x4*>(wl + j * kTile + ((sb & 3) * 16));
#pragma unroll
            for (int j = 0; j < 2; j++) {
                // (the two fp16 of the header forced into the normal range, so that the units stay finite)
                const uint32_t dw0 = (hd[j][0] & 0x03ff03ffu) | 0x2c002c00u, s0 = hd[j][1], s1 = hd[j][2], s2 = hd[j][3];
                const half2_t dd = __builtin_bit_cast(half2_t, dw0);
                const float d = (float)dd.x, dmin = (float)dd.y;
                const bool live = d != 0.f;
                sc4[j][0] = live ? s0 & 0x3F3F3F3Fu : 0u;
                sc4[j][1] = live ? (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u) : 0u;
                mn4[j][0] = s1 & 0x3F3F3F3Fu;
                mn4[j][1] = ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u);
                const int e_d = (int)((__float_as_uint(d) >> 23) & 0xFFu), e_m = (int)((__float_as_uint(dmin) >> 23) & 0xFFu);
                const int pw = live ? min(max(e_m - e_d - 10, 0), 10) : 0;
                sc_unit[j] = __uint_as_float((uint32_t)(127 + 10 - pw) << 23);
                const float cs_new = live ? d * __uint_as_float((uint32_t)(127 + 14 + pw) << 23) : (dmin != 0.f ? fabsf(dmin) * 512.0f : cs[j]);
                const float inv = 1.0f / cs_new, ratio = cs[j] * inv;
                min_unit[j] = fminf(fmaxf(-dmin * inv * 4096.0f, -1023.f), 1023.f);
                cs[j] = cs_new;
                if (PARTS & 16) {
#pragma unroll
                    for (int i = 0; i < MT; i++)
#pragma unroll
                        for (int x = 0; x < 16; x++) acc[i][j][x] *= ratio;
                }
            }
        }
        load_q(0, q);
        scales(0);
        if (DEC) {
            decode(0, fbn);
        } else {
            fbn[0] = __builtin_bit_cast(half8_t, q[0]), fbn[1] = __builtin_bit_cast(half8_t, q[1]);
        }
#pragma unroll
        for (int cc = 0; cc < 4; cc++) {
            if (cc < 3 && DEC) load_q(cc + 1, qn);
#pragma unroll
            for (int s = 0; s < 4; s++) {
                fb[0] = fbn[0], fb[1] = fbn[1];
                if (DEC) {
                    if (s < 3) {
                        decode(s + 1, fbn);
                    } else if (cc < 3) {
                        q[0] = qn[0], q[1] = qn[1];
                        if (PARTS & 2) scales(cc + 1);
                        decode(0, fbn);
                    }
                }
                const int step = 4 * cc + s, slot = step & 7;
#pragma unroll
                for (int i = 0; i < MT; i++) {
                    const half8_t fa = __builtin_bit_cast(half8_t, a[slot][i]);
#pragma unroll
                    for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa, fb[j], acc[i][j], 0, 0, 0);
                }
                if (PARTS & 4) {
                    __builtin_amdgcn_sched_barrier(0);
                    afetch(16 * sb + step + 8, slot);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        if (PARTS & 32) {
#pragma unroll
            for (int j = 0; j < 2; j++) {
                half8_t vh, vl;
#pragma unroll
                for (int s = 0; s < 8; s++) {
                    _Float16 hi, lo;
                    skn_split_hilo(min_unit[j] * byte_f(mn4[j][s >> 2], s & 3), hi, lo);
                    vh[s] = hi, vl[s] = lo;
                }
#pragma unroll
                for (int i = 0; i < MT; i++) {
                    const half8_t fs = __builtin_bit_cast(half8_t, a[i][0]);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fs, vh, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fs, vl, acc[i][j], 0, 0, 0);
                }
            }
        }
    }
    float s = cs[0] + cs[1] + min_unit[0] + min_unit[1] + (float)(mn4[0][0] ^ mn4[1][1] ^ mn4[0][1] ^ mn4[1][0]);
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int x = 0; x < 16; x++) s += acc[i][j][x];
    out[blockIdx.x * 512 + tid] = s;
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

// ns per k-step and SIMD (two wavefronts, eight matrix instructions) of the model of the Q4_K GEMM loop with the given
// parts (see q4k_loop_kernel; built: 0, 3, 4, 7, 15, 31, 47, 55, 59, 63).  data_dev: 64 MiB of device memory whose
// content does not matter, scratch_dev: 512 KiB.
extern "C" int skn_test_q4k_gemm_loop(skn_ctx* ctx, int parts, const void* data_dev, float* scratch_dev, double* ns_out) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_test_q4k_gemm_loop: ctx is null");
    SKN_REQUIRE(ctx, data_dev && scratch_dev && ns_out && ((uintptr_t)data_dev & 15) == 0, SKN_ERR_ARG,
                "skn_test_q4k_gemm_loop: bad arguments");
    const int superblocks = 64, grid = ctx->compute_units;
    SKN_REQUIRE(ctx, grid * 512 * sizeof(float) <= 512 * 1024, SKN_ERR_SHAPE, "skn_test_q4k_gemm_loop: scratch too small");
    const u32x4* a = (const u32x4*)data_dev;
    const uint32_t a_bytes = 64u << 20;
    double us = 0.0;
    int rc;
#define SKN_CASE(P)                                                                                                       \
    case P:                                                                                                               \
        rc = time_launches(ctx, 3, [&] { skn_launch(ctx, q4k_loop_kernel<P>, dim3(grid), dim3(512), 0, a, a_bytes, scratch_dev, superblocks, 1u); }, &us); \
        break;
    switch (parts) {
        SKN_CASE(0) SKN_CASE(3) SKN_CASE(4) SKN_CASE(7) SKN_CASE(15) SKN_CASE(31) SKN_CASE(47) SKN_CASE(55) SKN_CASE(59) SKN_CASE(63)
        default: return skn_fail(ctx, SKN_ERR_ARG, "skn_test_q4k_gemm_loop: the combination of parts %d is not built", parts);
    }
#undef SKN_CASE
    if (rc != SKN_OK) return rc;
    *ns_out = us * 1e3 / (superblocks * 16.0);
    return SKN_OK;
}
