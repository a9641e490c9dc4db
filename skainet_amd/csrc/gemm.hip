// Batched quantized GEMM  C[m,n] = sum_k A[m,k] * deq(W)[n,k]  (A bf16 [m,k], W GGUF blocks [n,k], C fp32 [m,n])
// on the matrix cores (v_mfma_f32_32x32x16_f16, fp32 accumulation).
//
// The tolerance asked of this op (1e-3 of max(|c|, 1e-3 * max|c|)) needs about 20 bits of every weight: a
// dequantized weight rounded to one fp16 / bf16 operand (11 / 8 bits) would miss it on outputs near zero.
// Both paths below therefore feed the MFMA with operands that are exact or exact to 2^-22:
//
//   * Activations: bf16 -> fp16 is exact for every value whose magnitude is within fp16's normal range; each
//     row is first scaled by a power of two that puts its largest magnitude just below 2^10 and the scale is
//     undone in the epilogue.  Products and sums are fp32 inside the MFMA.  Both paths read them in "fragment
//     order" (see prep_a_frag_kernel): a matrix-instruction operand is one coalesced 1 KiB load, no LDS.
//   * Weights, general path (every format but Q4_K): W is dequantized once into a workspace as an fp16 pair
//     hi = f16(w), lo = f16((w - hi) * 2^11) (hi + lo * 2^-11 = w to 2^-22 relative, or 2^-36 absolute for
//     weights in fp16's subnormal range), also in fragment order; each k-step issues two MFMAs per tile into two
//     sets of accumulators that are combined at the end.
//   * Weights, Q4_K path: see gemm_q4k_frag_kernel -- the 4-bit quants times their 6-bit sub-block scale are
//     integers below 2^10, exact in fp16, so one MFMA per k-step suffices; the f16 superblock scale d is the
//     unit in which a column's accumulators are kept.
#include "common.h"
#include "gemm_q6k.h"

#include <type_traits>

namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kBN = 64;   // workgroup tile columns (weight rows)

// C tile store: acc register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32 of the 32x32 tile
__device__ __forceinline__ void store_tile(const float16_t& acc, float* __restrict__ c, int ldc, int row0, int col0,
                                           int m, int n, const float* __restrict__ inv_scale, int lane,
                                           bool accumulate = false) {
    const int col = col0 + (lane & 31);
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int row = row0 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (row < m && col < n) {
            float* dst = c + (size_t)row * ldc + col;
            *dst = accumulate ? *dst + acc[r] * inv_scale[row] : acc[r] * inv_scale[row];
        }
    }
}

// the same with the sixteen row scales in hand (sc[r]: the scale of the row that register r holds)
__device__ __forceinline__ void store_tile_scaled(const float16_t& acc, float* __restrict__ c, int ldc, int row0, int col0,
                                                  int m, int n, const float (&sc)[16], int lane, bool accumulate) {
    const int col = col0 + (lane & 31);
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int row = row0 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (row < m && col < n) {
            float* dst = c + (size_t)row * ldc + col;
            *dst = accumulate ? *dst + acc[r] * sc[r] : acc[r] * sc[r];
        }
    }
}

// ---- Q4_K path: weights unpacked in the kernel, one MFMA per k-step, operands loaded by the wavefronts ------
// Workgroup of eight wavefronts, tile (64 MT) x 64.  The tile is divided in two along m; along k it is not
// divided spatially but by superblock: wavefront (mh, kq) computes rows [32 MT mh, 32 MT (mh + 1)) x all 64
// columns for superblocks kq, kq + 4, ..., and the four partial tiles of each half are added through LDS at
// the end.  The activations are prepared in "fragment order": for a block of 32 rows, a 64-element chunk and a
// k-step s, the 64 x 16 bytes that the 64 lanes feed to one matrix instruction are contiguous (lane l = 32 h + r
// holds row r and the eight elements that nibble dword 4 h + s of the chunk unpacks to), so a fragment is one
// coalesced 1 KiB load and never passes through LDS.  The weights of four superblocks (576 contiguous bytes of
// each of the 64 rows) are copied from global memory straight into LDS once per group of four superblocks --
// the only barrier in the loop -- from where each lane picks the 16 bytes of its row and k-step quartet.
// w[n, 256 b + e] = d * (sc_j * q) - dmin * m_j  (j = sub-block of e).  sc_j * q is an integer below 2^10: the
// nibble masked in place is the fp16 subnormal q * 2^-24 (or 16 q * 2^-24 for a high nibble) and one packed
// fp16 multiply by sc_j * 2^10 (or sc_j * 2^6) gives sc_j * q * 2^-14 exactly -- an fp16 operand the matrix
// core takes as is.  One set of accumulators: see the kernel.
// LDS pitch of a weight row: the 576 bytes of four superblocks plus one sixteen-byte pad piece.  With 576 (144 dwords,
// 16 mod 64) rows r, r + 4, r + 8, ... start in the same bank and the 128-bit reads of a wavefront's 32 rows were
// eight-fold bank conflicts; with 592 (148 dwords, 20 mod 64) sixteen consecutive rows tile all 64 banks.
constexpr int kWPieces = 37;
constexpr int kWPitch = kWPieces * 16;

// Activations bf16 [m, k] -> fragment order.  One workgroup per R rows of the padded row count (rows >= m are
// zero), one wavefront per row: the row's largest magnitude fixes its power-of-two scale, then the row is
// converted 4096 elements at a time into LDS, laid out so that the copy to global memory writes runs of 16 R
// bytes (the same sixteen bytes of R neighbouring rows).
// afrag: [row block][chunk][k-step][lane] x 8 halves.  sfrag: [row block][superblock][lane] x 8 halves: the eight
// sub-block sums of row r times 2^-12 as fp16 pairs, lanes 0..31 the "hi" parts, lanes 32..63 the "lo" parts
// (SUMS; k must then be a multiple of 256).
// The rows come from a source (skn_gemm_src): bf16 as given; fp32 rounded to bf16 (nearest even) on the way in;
// or fp32 RMS-normalized first (x * r * g, r = 1 / sqrt(mean(x^2) + eps)) -- the row-wise kernel that would
// otherwise run before the GEMM.
struct PrepRow {
    const void* a;   // the row
    const void* b;   // SKN_SRC_RMSNORM: the norm weights
    float r;         // SKN_SRC_RMSNORM: 1 / sqrt(mean(x^2) + eps)
};

__device__ __forceinline__ uint32_t bf16_rne(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

// elements [i, i + 4) of the row as four bf16 bit patterns in two words
template <int SRC>
__device__ __forceinline__ void load_bf16x4(const PrepRow& row, int i, uint32_t& lo, uint32_t& hi) {
    if (SRC == SKN_SRC_BF16) {
        const u32x2 v = *reinterpret_cast<const u32x2*>((const uint16_t*)row.a + i);
        lo = v.x, hi = v.y;
        return;
    }
    const float4 x = *reinterpret_cast<const float4*>((const float*)row.a + i);
    float y[4] = {x.x, x.y, x.z, x.w};
    if (SRC == SKN_SRC_RMSNORM) {
        const float4 g = *reinterpret_cast<const float4*>((const float*)row.b + i);
        y[0] = x.x * row.r * g.x, y[1] = x.y * row.r * g.y, y[2] = x.z * row.r * g.z, y[3] = x.w * row.r * g.w;
    }
    lo = bf16_rne(y[0]) | (bf16_rne(y[1]) << 16);
    hi = bf16_rne(y[2]) | (bf16_rne(y[3]) << 16);
}

template <int R, int SRC, bool SUMS>
__global__ __launch_bounds__(64 * R) void prep_a_frag_kernel(const skn_gemm_src src, _Float16* __restrict__ afrag,
                                                            float* __restrict__ inv_scale, _Float16* __restrict__ sfrag,
                                                            int m, int k) {
    __shared__ __align__(16) u32x4 stage[512 * R];  // [chunk 64][k-step 4][half 2][row R] sixteen-byte pieces
    const int tid = threadIdx.x, lane = tid & 63, r8 = tid >> 6;
    const int row = blockIdx.x * R + r8;
    const bool real = row < m;
    const size_t row_off = (size_t)(real ? row : 0) * k;
    PrepRow ar;
    ar.a = SRC == SKN_SRC_BF16 ? (const void*)((const uint16_t*)src.a + row_off) : (const void*)((const float*)src.a + row_off);
    ar.b = src.b;
    ar.r = 1.f;
    if (SRC == SKN_SRC_RMSNORM) {
        const float* xr = (const float*)ar.a;
        float ss = 0.f;
        for (int i0 = 0; i0 < (k >> 2); i0 += 512) {
            float4 v[8];
#pragma unroll
            for (int j = 0; j < 8; j++) v[j] = reinterpret_cast<const float4*>(xr)[min(i0 + lane + 64 * j, (k >> 2) - 1)];
#pragma unroll
            for (int j = 0; j < 8; j++)
                if (i0 + lane + 64 * j < (k >> 2)) ss += (v[j].x * v[j].x + v[j].y * v[j].y) + (v[j].z * v[j].z + v[j].w * v[j].w);
        }
        ss = wave_sum(ss);
        ar.r = 1.0f / sqrtf(ss / (float)k + src.eps);
    }
    const int nch = k >> 6, nb = k >> 8;
    auto widen = [](uint32_t pair, int which) { return __uint_as_float(which ? pair & 0xFFFF0000u : pair << 16); };

    // pass 1: the row's largest finite magnitude
    float mx = 0.f;
    for (int i0 = 0; i0 < (k >> 3); i0 += 512) {  // eight loads in flight per lane
        u32x4 v[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int i = 8 * min(i0 + lane + 64 * j, (k >> 3) - 1);
            uint32_t w0, w1, w2, w3;
            load_bf16x4<SRC>(ar, i, w0, w1);
            load_bf16x4<SRC>(ar, i + 4, w2, w3);
            v[j] = u32x4{w0, w1, w2, w3};
        }
#pragma unroll
        for (int j = 0; j < 8; j++)
#pragma unroll
            for (int x = 0; x < 8; x++) {
                const float f = fabsf(widen(v[j][x >> 1], x & 1));
                if (f == f && f < INFINITY) mx = fmaxf(mx, f);
            }
    }
    mx = wave_max(mx);
    if (!real) mx = 0.f;
    int e = 9;  // a zero row keeps scale 1
    if (mx > 0.f) e = (int)((__float_as_uint(mx) >> 23) & 0xFF) - 127;
    e = max(e, -100);  // (a subnormal maximum: exponent field 0)
    const float scale = real ? __uint_as_float((uint32_t)(127 + 9 - e) << 23) : 0.f;
    if (lane == 0 && real) inv_scale[row] = __uint_as_float((uint32_t)(127 - 9 + e) << 23);
    const int mb = row >> 5, r = row & 31;

    // pass 2: slabs of 4096 elements = 64 chunks = 512 tasks (chunk c, nibble dword dw), eight per lane
    for (int k0 = 0; k0 < k; k0 += 4096) {
        const int tasks = min(4096, k - k0) >> 3;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int task = lane + 64 * j;
            const int c = task >> 3, dw = task & 7;
            uint2 lo = make_uint2(0u, 0u), hi = lo;
            if (task < tasks) {
                load_bf16x4<SRC>(ar, k0 + 64 * c + 4 * dw, lo.x, lo.y);
                load_bf16x4<SRC>(ar, k0 + 64 * c + 32 + 4 * dw, hi.x, hi.y);
            }
            _Float16 l[4], u[4];
            l[0] = (_Float16)(widen(lo.x, 0) * scale), l[1] = (_Float16)(widen(lo.x, 1) * scale);
            l[2] = (_Float16)(widen(lo.y, 0) * scale), l[3] = (_Float16)(widen(lo.y, 1) * scale);
            u[0] = (_Float16)(widen(hi.x, 0) * scale), u[1] = (_Float16)(widen(hi.x, 1) * scale);
            u[2] = (_Float16)(widen(hi.y, 0) * scale), u[3] = (_Float16)(widen(hi.y, 1) * scale);
            float sl = ((float)l[0] + (float)l[1]) + ((float)l[2] + (float)l[3]);
            float su = ((float)u[0] + (float)u[1]) + ((float)u[2] + (float)u[3]);
            // totals over the eight lanes of the chunk
            sl += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(sl), 0xB1, 0xF, 0xF, true));
            su += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(su), 0xB1, 0xF, 0xF, true));
            sl += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(sl), 0x4E, 0xF, 0xF, true));
            su += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(su), 0x4E, 0xF, 0xF, true));
            sl += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(sl), 0x141, 0xF, 0xF, true));
            su += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(su), 0x141, 0xF, 0xF, true));
            half8_t o;
            o[0] = l[0], o[1] = l[2], o[2] = u[0], o[3] = u[2], o[4] = l[1], o[5] = l[3], o[6] = u[1], o[7] = u[3];
            const int h = dw >> 2, s = dw & 3;
            stage[((c * 4 + s) * 2 + h) * R + r8] = __builtin_bit_cast(u32x4, o);
            if (SUMS && dw == 0 && task < tasks) {
                _Float16 h0, h1, l0, l1;
                skn_split_hilo(sl * 0x1p-12f, h0, l0);
                skn_split_hilo(su * 0x1p-12f, h1, l1);
                const int cg = (k0 >> 6) + c;
                _Float16* sf = sfrag + ((size_t)mb * nb + (cg >> 2)) * 512 + 2 * (cg & 3);
                half2_t vh = {h0, h1}, vl = {l0, l1};
                *reinterpret_cast<half2_t*>(sf + r * 8) = vh;
                *reinterpret_cast<half2_t*>(sf + (32 + r) * 8) = vl;
            }
        }
        __syncthreads();
        // piece i = ((c 4 + s) 2 + h) R + row: R consecutive lanes write 16 R contiguous bytes
        u32x4* out = reinterpret_cast<u32x4*>(afrag) + ((size_t)mb * nch + (k0 >> 6)) * 256 + (blockIdx.x % (32 / R)) * R;
#pragma unroll
        for (int it = 0; it < 8; it++) {
            const int i = tid + 64 * R * it, csh = i / R;
            if (csh < tasks) out[(size_t)(csh >> 1) * 64 + (csh & 1) * 32 + (i % R)] = stage[i];
        }
        __syncthreads();
    }
}

// The same preparation with a row spread over two wavefronts (k <= 16384): every element is read from memory once and
// stays in registers through the three steps that the one-wavefront-per-row kernel above makes three passes for (sum of
// squares, largest magnitude, conversion), two rows per workgroup, twice as many workgroups.  Thread t of a row takes
// tasks t, t + 128, ... (task = chunk c, nibble dword dw: four elements at 64 c + 4 dw and four at 64 c + 32 + 4 dw);
// its sixteen-byte pieces go straight to their place in the fragment order.  Consecutive row pairs go to workgroups of
// one XCD (blockIdx % 8), so that the 128-byte lines they share are completed in one L2.
template <int NT, int SRC, bool SUMS>
__global__ __launch_bounds__(256) void prep_a_rows_kernel(const skn_gemm_src src, _Float16* __restrict__ afrag,
                                                         float* __restrict__ inv_scale, _Float16* __restrict__ sfrag,
                                                         int m, int k) {
    __shared__ float red_ss[2][2], red_mx[2][2];
    const int tid = threadIdx.x, t = tid & 127, rw = tid >> 7, wv = (tid >> 6) & 1;
    const int n_pairs = gridDim.x, per_xcd = n_pairs >> 3;
    const int pair = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    const int row = 2 * pair + rw;
    const bool real = row < m;
    const size_t row_off = (size_t)(real ? row : 0) * k;
    const int tasks = k >> 3, nch = k >> 6, nb = k >> 8;
    const float* xf = (const float*)src.a + row_off;
    const uint16_t* xb = (const uint16_t*)src.a + row_off;
    float v[NT][8];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < NT; j++) {
        const int task = min(t + 128 * j, tasks - 1), c = task >> 3, dw = task & 7;
        const int e0 = 64 * c + 4 * dw;
        if (SRC == SKN_SRC_BF16) {
            const u32x2 lo = *reinterpret_cast<const u32x2*>(xb + e0), hi = *reinterpret_cast<const u32x2*>(xb + e0 + 32);
            v[j][0] = __uint_as_float(lo.x << 16), v[j][1] = __uint_as_float(lo.x & 0xFFFF0000u);
            v[j][2] = __uint_as_float(lo.y << 16), v[j][3] = __uint_as_float(lo.y & 0xFFFF0000u);
            v[j][4] = __uint_as_float(hi.x << 16), v[j][5] = __uint_as_float(hi.x & 0xFFFF0000u);
            v[j][6] = __uint_as_float(hi.y << 16), v[j][7] = __uint_as_float(hi.y & 0xFFFF0000u);
        } else {
            const float4 lo = *reinterpret_cast<const float4*>(xf + e0), hi = *reinterpret_cast<const float4*>(xf + e0 + 32);
            v[j][0] = lo.x, v[j][1] = lo.y, v[j][2] = lo.z, v[j][3] = lo.w;
            v[j][4] = hi.x, v[j][5] = hi.y, v[j][6] = hi.z, v[j][7] = hi.w;
            if (SRC == SKN_SRC_RMSNORM && t + 128 * j < tasks)
                ss += ((lo.x * lo.x + lo.y * lo.y) + (lo.z * lo.z + lo.w * lo.w)) + ((hi.x * hi.x + hi.y * hi.y) + (hi.z * hi.z + hi.w * hi.w));
        }
    }
    float r = 1.f;
    if (SRC == SKN_SRC_RMSNORM) {
        ss = wave_sum(ss);
        if ((tid & 63) == 0) red_ss[rw][wv] = ss;
        __syncthreads();
        r = 1.0f / sqrtf((red_ss[rw][0] + red_ss[rw][1]) / (float)k + src.eps);
    }
    // the bf16 values the GEMM is defined on (fp32 sources: rounded to nearest even here), and their largest magnitude
    float mx = 0.f;
#pragma unroll
    for (int j = 0; j < NT; j++) {
        if (SRC != SKN_SRC_BF16) {
            const int task = min(t + 128 * j, tasks - 1), c = task >> 3, dw = task & 7;
            float4 glo = make_float4(1.f, 1.f, 1.f, 1.f), ghi = glo;
            if (SRC == SKN_SRC_RMSNORM) {
                glo = *reinterpret_cast<const float4*>((const float*)src.b + 64 * c + 4 * dw);
                ghi = *reinterpret_cast<const float4*>((const float*)src.b + 64 * c + 32 + 4 * dw);
            }
            const float g[8] = {glo.x, glo.y, glo.z, glo.w, ghi.x, ghi.y, ghi.z, ghi.w};
#pragma unroll
            for (int x = 0; x < 8; x++) {
                const float y = SRC == SKN_SRC_RMSNORM ? v[j][x] * r * g[x] : v[j][x];
                v[j][x] = __uint_as_float(bf16_rne(y) << 16);
            }
        }
#pragma unroll
        for (int x = 0; x < 8; x++) {
            const float f = fabsf(v[j][x]);
            if (f == f && f < INFINITY) mx = fmaxf(mx, f);
        }
    }
    mx = wave_max(mx);
    if ((tid & 63) == 0) red_mx[rw][wv] = mx;
    __syncthreads();
    mx = real ? fmaxf(red_mx[rw][0], red_mx[rw][1]) : 0.f;
    int e = 9;  // a zero row keeps scale 1
    if (mx > 0.f) e = (int)((__float_as_uint(mx) >> 23) & 0xFF) - 127;
    e = max(e, -100);
    const float scale = real ? __uint_as_float((uint32_t)(127 + 9 - e) << 23) : 0.f;
    if (t == 0 && real) inv_scale[row] = __uint_as_float((uint32_t)(127 - 9 + e) << 23);
    const int mb = row >> 5, rr = row & 31;
    u32x4* out = reinterpret_cast<u32x4*>(afrag) + (size_t)mb * nch * 256 + rr;
#pragma unroll
    for (int j = 0; j < NT; j++) {
        const int task = t + 128 * j, c = task >> 3, dw = task & 7;
        _Float16 l[4], u[4];
#pragma unroll
        for (int x = 0; x < 4; x++) l[x] = (_Float16)(v[j][x] * scale), u[x] = (_Float16)(v[j][4 + x] * scale);
        float sl = ((float)l[0] + (float)l[1]) + ((float)l[2] + (float)l[3]);
        float su = ((float)u[0] + (float)u[1]) + ((float)u[2] + (float)u[3]);
        if (SUMS) {  // totals over the eight lanes of the chunk
            sl += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(sl), 0xB1, 0xF, 0xF, true));
            su += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(su), 0xB1, 0xF, 0xF, true));
            sl += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(sl), 0x4E, 0xF, 0xF, true));
            su += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(su), 0x4E, 0xF, 0xF, true));
            sl += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(sl), 0x141, 0xF, 0xF, true));
            su += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(su), 0x141, 0xF, 0xF, true));
        }
        if (task < tasks) {
            half8_t o;
            o[0] = l[0], o[1] = l[2], o[2] = u[0], o[3] = u[2], o[4] = l[1], o[5] = l[3], o[6] = u[1], o[7] = u[3];
            const int h = dw >> 2, sq = dw & 3;
            out[((size_t)c * 4 + sq) * 64 + h * 32] = __builtin_bit_cast(u32x4, o);
            if (SUMS && dw == 0) {
                _Float16 h0, h1, l0, l1;
                skn_split_hilo(sl * 0x1p-12f, h0, l0);
                skn_split_hilo(su * 0x1p-12f, h1, l1);
                _Float16* sf = sfrag + ((size_t)mb * nb + (c >> 2)) * 512 + 2 * (c & 3);
                half2_t vh = {h0, h1}, vl = {l0, l1};
                *reinterpret_cast<half2_t*>(sf + rr * 8) = vh;
                *reinterpret_cast<half2_t*>(sf + (32 + rr) * 8) = vl;
            }
        }
    }
}

template <int SRC, bool SUMS>
void launch_prep(skn_ctx* ctx, const skn_gemm_src& src, _Float16* afrag, float* isc, _Float16* sfrag, int m, int m_pad, int k) {
    // (m_pad is a multiple of 32: the pair count divides by the eight XCDs its workgroups are dealt to)
    if (k <= 16384 && m_pad % 16 == 0) {
        const dim3 grid(m_pad / 2), block(256);
        const int nt = (k / 8 + 127) / 128;
        if (nt <= 4) skn_launch(ctx, prep_a_rows_kernel<4, SRC, SUMS>, grid, block, 0, src, afrag, isc, sfrag, m, k);
        else if (nt <= 8) skn_launch(ctx, prep_a_rows_kernel<8, SRC, SUMS>, grid, block, 0, src, afrag, isc, sfrag, m, k);
        else if (nt <= 12) skn_launch(ctx, prep_a_rows_kernel<12, SRC, SUMS>, grid, block, 0, src, afrag, isc, sfrag, m, k);
        else skn_launch(ctx, prep_a_rows_kernel<16, SRC, SUMS>, grid, block, 0, src, afrag, isc, sfrag, m, k);
    } else {
        skn_launch(ctx, prep_a_frag_kernel<4, SRC, SUMS>, dim3(m_pad / 4), dim3(256), 0, src, afrag, isc, sfrag, m, k);
    }
}

// up to three weight matrices [n_i, k] multiplied by the same activations in one launch
struct Q4kFragSegs {
    const uint8_t* w[3];
    float* c[3];
    int n[3];
    int accumulate[3];  // add to c instead of overwriting it
    int tile0[3];       // first column tile of each matrix (unused entries: n_tiles)
    int n_tiles;
    // pair != 0: w[0], w[1] are the gate and up matrices of a SwiGLU; a tile holds the same 32 columns of both
    // (its two 32-column halves) and stores silu(gate) * up into c[0]
    int pair;
};

// the kernel's LDS (weight buffers, then the tile exchange) exceeds the static limit (the scales of the tile's rows follow it): dynamic, opted in per
// device by skn_gemm_init
template <int MT, int MH>
constexpr int frag_lds_bytes() {
    return 2 * kBN * kWPitch > MT * MH * 24576 ? 2 * kBN * kWPitch : MT * MH * 24576;
}

// Accumulators: acc holds the running sum of a column in units of cs = d * 2^14 of the latest superblock whose d
// is not zero.  Entering a superblock it is rescaled by cs_old / cs_new (a relative error of 2^-23 per
// superblock, against the 1e-3 asked of the op); the superblock's integer products then add to it as they come
// out of the matrix core, and so does the "- dmin * m_j" term: one more sixteen-deep product per tile between
// the activation sub-block sums (fp16 hi | lo) and -(dmin / cs) * m_j * 2^12, itself split into an fp16 pair.
template <int MT, int MH>
__global__ __launch_bounds__(256 * MH) __attribute__((amdgpu_waves_per_eu(2, 2)))
void gemm_q4k_frag_kernel(const u32x4* __restrict__ afrag, const u32x4* __restrict__ sfrag, const Q4kFragSegs segs,
                          const float* __restrict__ inv_scale, int m, int k, uint32_t a_bytes) {
    constexpr int kWBuf = kBN * kWPitch;
    extern __shared__ __align__(16) uint8_t lds[];  // max(2 kWBuf, MT x 48 KiB) bytes
    const int tid = threadIdx.x, lane = tid & 63;
    // (the wavefront's index as a scalar: everything derived from it -- its row blocks, its superblocks, the
    // base addresses of its fragments -- then lives in scalar registers, and a fragment load is scalar base +
    // lane offset instead of a 64-bit vector add per load)
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kq = wave & 3, mh = wave >> 2;
    const int h = lane >> 5, r = lane & 31;
    const int nb = k >> 8, nch = k >> 6, groups = (nb + 3) >> 2;
    // tile -> (row tile, weight matrix, column tile): the column tiles of up to three matrices sharing the
    // activations are laid side by side
    const int mt = blockIdx.x / segs.n_tiles, tn = blockIdx.x - mt * segs.n_tiles;
    const bool pair = segs.pair != 0;
    const int seg = pair ? 0 : (tn >= segs.tile0[2] ? 2 : (tn >= segs.tile0[1] ? 1 : 0));
    const uint8_t* __restrict__ w = segs.w[seg];
    float* __restrict__ c = segs.c[seg];
    const int n = segs.n[seg];
    const int mb0 = (MH * mt + mh) * MT, n0 = pair ? tn * 32 : (tn - segs.tile0[seg]) * kBN;

    // Weight staging, global memory straight into LDS: a wavefront-wide load fills 64 sixteen-byte slots
    // i * 64 + lane; slot P holds piece P % 37 of tile row P / 37 (36 pieces = the 576 bytes of four
    // superblocks, the 37th a pad that repeats the last).  The 37 loads of a group are dealt round the wavefronts.  Completion is waited for
    // with the vector-memory counter before the barrier that publishes the buffer.
    auto wfetch = [&](int g, int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int x = 0; x < (kWPieces + 4 * MH - 1) / (4 * MH); x++) {
            const int i = wave + 4 * MH * x;
            if (i < kWPieces) {
                const int p = i * 64 + lane, row = p / kWPieces, col = min(p - kWPieces * row, 35);
                const int off = min(g * 576 + col * 16, nb * 144 - 16);  // (a short last group repeats the row's last piece)
                const uint8_t* wsrc = pair && row >= 32 ? segs.w[1] : w;  // (pair: tile rows 32.. are the up matrix)
                const uint8_t* src = wsrc + (size_t)min(n0 + (pair ? row & 31 : row), n - 1) * nb * 144 + off;
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                                 (__attribute__((address_space(3))) void*)(lds + buf * kWBuf + i * 1024), 16, 0, 0);
            }
        }
    };

    // The activation fragments are read with buffer loads: a scalar byte offset (row block, k-step) plus the
    // lane's sixteen bytes, no vector address arithmetic per load.
    const __amdgpu_buffer_rsrc_t arsrc = __builtin_amdgcn_make_buffer_rsrc((void*)afrag, 0, (int)a_bytes, 0x00020000);
    uint32_t abase[MT];  // byte offset of the row block's first fragment
#pragma unroll
    for (int i = 0; i < MT; i++) abase[i] = (uint32_t)(mb0 + i) * (uint32_t)nch * 4096u;
    // activation fragments: a ring of eight k-steps; the slot of step t is refilled with step t + 8 as soon as
    // the matrix instructions of step t are issued
    u32x4 a[8][MT];
    auto afetch = [&](int step, int slot) __attribute__((always_inline)) {  // step: 16 per superblock, absolute
#pragma unroll
        for (int i = 0; i < MT; i++)
            a[slot][i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(arsrc, lane * 16, (int)(abase[i] + (uint32_t)step * 1024u), 0));
    };
    float16_t acc[MT][2];
    float cs[2] = {1.f, 1.f};
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int x = 0; x < 16; x++) acc[i][j][x] = 0.f;

    // the scales of the tile's rows, for the store at the end
    float* isc_lds = reinterpret_cast<float*>(lds + frag_lds_bytes<MT, MH>());
    wfetch(0, 0);
    if (tid < 32 * MT * MH) isc_lds[tid] = inv_scale[MH * mt * MT * 32 + tid];
    if (kq < nb) {
        // (the first eight fragment steps are requested behind the weights and stay in flight past the barrier)
#pragma unroll
        for (int s = 0; s < 8; s++) afetch(16 * kq + s, s);
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(8 * MT) : "memory");
    } else {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

    for (int g = 0; g < groups; g++) {
        const int sb = 4 * g + kq;
        if (g + 1 < groups) wfetch(g + 1, (g + 1) & 1);
        if (sb < nb) {
            // this lane's weight rows (one per 32-column tile): the 144 bytes of superblock sb
            const uint8_t* wl = lds + (g & 1) * kWBuf + r * kWPitch + kq * 144;
            constexpr int kTile = 32 * kWPitch;  // the lane's row of the second 32-column tile
            u32x4 hd[2], sf[MT];
#pragma unroll
            for (int j = 0; j < 2; j++) hd[j] = *reinterpret_cast<const u32x4*>(wl + j * kTile);
            // The eight 6-bit scales and mins of the superblock, four to a word: bytes 0..3 of the twelve hold the
            // low scales, 4..7 the low mins, 8..11 the low nibbles of the high ones, whose top two bits sit in
            // bits 6..7 of the first eight bytes.
            uint32_t sc4[2][2], mn4[2][2];
            float min_unit[2], sc_unit[2];
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const uint32_t dw0 = hd[j][0], s0 = hd[j][1], s1 = hd[j][2], s2 = hd[j][3];
                const half2_t dd = __builtin_bit_cast(half2_t, dw0);
                const float d = (float)dd.x, dmin = (float)dd.y;
                const bool live = d != 0.f;  // (a zero d: the products are zeroed)
                sc4[j][0] = live ? s0 & 0x3F3F3F3Fu : 0u;
                sc4[j][1] = live ? (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u) : 0u;
                mn4[j][0] = s1 & 0x3F3F3F3Fu;
                mn4[j][1] = ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u);
                // The unit is d * 2^(14 + p) and the weight operands are sc * q * 2^-(14 + p) -- exact in fp16 for
                // p <= 10.  p = 0 unless |dmin / d| is so large (>= 2^11) that the min operands below would
                // overflow fp16; beyond 2^21 they saturate.
                const int e_d = (int)((__float_as_uint(d) >> 23) & 0xFFu), e_m = (int)((__float_as_uint(dmin) >> 23) & 0xFFu);
                const int pw = live ? min(max(e_m - e_d - 10, 0), 10) : 0;
                sc_unit[j] = __uint_as_float((uint32_t)(127 + 10 - pw) << 23);
                // (no live weights: the unit is free, and taken from dmin so that the min operands are well inside
                // fp16 -- the unit inherited from the last live superblock can be orders of magnitude off)
                const float cs_new = live ? d * __uint_as_float((uint32_t)(127 + 14 + pw) << 23)
                                          : (dmin != 0.f ? fabsf(dmin) * 512.0f : cs[j]);
                const float inv = 1.0f / cs_new, ratio = cs[j] * inv;
                // -(dmin / unit) * 2^12: times a min (< 64) it stays inside fp16
                min_unit[j] = fminf(fmaxf(-dmin * inv * 4096.0f, -1023.f), 1023.f);
                cs[j] = cs_new;
#pragma unroll
                for (int i = 0; i < MT; i++)
#pragma unroll
                    for (int x = 0; x < 16; x++) acc[i][j][x] *= ratio;
            }
            auto byte_f = [](uint32_t word, int b) { return (float)((word >> (8 * b)) & 0xFFu); };
            // Sixteen k-steps, software-pipelined: the weight fragments of step t + 1 are unpacked (vector ALU)
            // while the matrix instructions of step t run.
            u32x4 q[2], qn[2];
            half2_t mul_lo[2], mul_hi[2];
            half8_t fb[2], fbn[2];
            auto load_q = [&](int cc, u32x4* dst) __attribute__((always_inline)) {
#pragma unroll
                for (int j = 0; j < 2; j++) dst[j] = *reinterpret_cast<const u32x4*>(wl + j * kTile + 16 + 32 * cc + 16 * h);
            };
            auto scales = [&](int cc) __attribute__((always_inline)) {  // sub-blocks 2 cc (low nibbles), 2 cc + 1 (high)
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const float fl = byte_f(sc4[j][cc >> 1], 2 * (cc & 1)) * sc_unit[j];
                    const float fh = byte_f(sc4[j][cc >> 1], 2 * (cc & 1) + 1) * (sc_unit[j] * 0.0625f);
                    mul_lo[j] = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_pkrtz(fl, fl));  // (six bits times a power of two: exact)
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
            load_q(0, q);
            scales(0);
            decode(0, fbn);
            auto chunk = [&](auto cc_const) __attribute__((always_inline)) {
                constexpr int cc = decltype(cc_const)::value;
                if (cc == 2) {
#pragma unroll
                    for (int i = 0; i < MT; i++) sf[i] = sfrag[((size_t)(mb0 + i) * nb + sb) * 64 + lane];
                }
                if (cc < 3) load_q(cc + 1, qn);
#pragma unroll
                for (int s = 0; s < 4; s++) {
                    fb[0] = fbn[0], fb[1] = fbn[1];
                    if (s < 3) {
                        decode(s + 1, fbn);
                    } else if (cc < 3) {
                        q[0] = qn[0], q[1] = qn[1];
                        scales(cc + 1);
                        decode(0, fbn);
                    }
                    const int step = 4 * cc + s, slot = step & 7;
#pragma unroll
                    for (int i = 0; i < MT; i++) {
                        const half8_t fa = __builtin_bit_cast(half8_t, a[slot][i]);
#pragma unroll
                        for (int j = 0; j < 2; j++)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa, fb[j], acc[i][j], 0, 0, 0);
                    }
                    // refill the slot: eight steps ahead in this superblock, or the first half of superblock sb + 4
                    // (past the end: a repeat of the last superblock, unused)
                    // (the refill stays here: moved further down by the scheduler, the ring would be shallower than it looks)
                    __builtin_amdgcn_sched_barrier(0);
                    afetch(step < 8 ? 16 * sb + step + 8 : 16 * min(sb + 4, nb - 1) + step - 8, slot);
                    __builtin_amdgcn_sched_barrier(0);
                }
            };
            chunk(std::integral_constant<int, 0>{});
            chunk(std::integral_constant<int, 1>{});
            chunk(std::integral_constant<int, 2>{});
            chunk(std::integral_constant<int, 3>{});
            // the "- dmin * m" term of the superblock
#pragma unroll
            for (int j = 0; j < 2; j++) {
                half8_t vh, vl;
#pragma unroll
                for (int s = 0; s < 8; s++) {
                    _Float16 a, b;
                    skn_split_hilo(min_unit[j] * byte_f(mn4[j][s >> 2], s & 3), a, b);
                    vh[s] = a, vl[s] = b;
                }
#pragma unroll
                for (int i = 0; i < MT; i++) {
                    const half8_t fs = __builtin_bit_cast(half8_t, sf[i]);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fs, vh, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fs, vl, acc[i][j], 0, 0, 0);
                }
            }
        }
        // a bare barrier: a full __syncthreads() would also wait for the fragment loads in flight
        // The next group's weights were requested before this superblock's 16 MT fragment loads, and loads
        // complete in order: once all but the newest 8 MT have landed, so have they.
        if (sb < nb) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(8 * MT) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }
    // back to true units
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int x = 0; x < 16; x++) acc[i][j][x] *= cs[j];

    // Add the four partial tiles of each half.  Tile t = 2 i + j belongs to wavefront kq = t % 4 of its half and
    // the other three hand theirs over.  Pair: the two column halves of row block i are needed together, so
    // wavefront i % 4 takes accumulator registers 0..7 of both and wavefront (i + 2) % 4 registers 8..15.
    float* red = reinterpret_cast<float*>(lds);
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int t = 2 * i + j;
#pragma unroll
            for (int xh = 0; xh < 2; xh++) {
                const int owner = pair ? (i + 2 * xh) & 3 : t & 3;
                if (kq != owner) {
                    float* dst = red + ((mh * 2 * MT + t) * 3 + ((kq - owner + 4) & 3) - 1) * 1024 + lane;
#pragma unroll
                    for (int x = 8 * xh; x < 8 * xh + 8; x++) dst[64 * x] = acc[i][j][x];
                }
            }
        }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < MT; i++) {
        if (pair) {
#pragma unroll
            for (int xh = 0; xh < 2; xh++)
                if (kq == ((i + 2 * xh) & 3)) {
                    const int col = n0 + (lane & 31);
#pragma unroll
                    for (int x = 8 * xh; x < 8 * xh + 8; x++) {
                        float g = acc[i][0][x], u = acc[i][1][x];
#pragma unroll
                        for (int o = 0; o < 3; o++) {
                            g += red[((mh * 2 * MT + 2 * i) * 3 + o) * 1024 + 64 * x + lane];
                            u += red[((mh * 2 * MT + 2 * i + 1) * 3 + o) * 1024 + 64 * x + lane];
                        }
                        // register x of lane l: row 8 (x / 4) + 4 (l / 32) + x % 4 of the 32 x 32 tile
                        const int row = (mb0 + i) * 32 + 8 * (x >> 2) + 4 * (lane >> 5) + (x & 3);
                        if (row < m && col < n) {
                            const float sc = isc_lds[row - MH * mt * MT * 32];
                            const float a = g * sc;
                            c[(size_t)row * n + col] = a / (1.0f + expf(-a)) * (u * sc);  // silu(gate) * up
                        }
                    }
                }
            continue;
        }
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int t = 2 * i + j;
            if (kq == (t & 3)) {
                float16_t sum = acc[i][j];
#pragma unroll
                for (int o = 0; o < 3; o++)
#pragma unroll
                    for (int x = 0; x < 16; x++) sum[x] += red[((mh * 2 * MT + t) * 3 + o) * 1024 + 64 * x + lane];
                float sc[16];
#pragma unroll
                for (int x = 0; x < 16; x++) sc[x] = isc_lds[(mh * MT + i) * 32 + 8 * (x >> 2) + 4 * (lane >> 5) + (x & 3)];
                store_tile_scaled(sum, c, n, (mb0 + i) * 32, n0 + 32 * j, m, n, sc, lane, segs.accumulate[seg] != 0);
            }
        }
    }
}


template <int MT, int MH>
int launch_frag(skn_ctx* ctx, int m_tiles, const u32x4* afrag, const u32x4* sfrag, const Q4kFragSegs& segs, const float* isc,
                int m, int k) {
    constexpr int kLds = frag_lds_bytes<MT, MH>() + 32 * MT * MH * 4;
    const uint32_t a_bytes = (uint32_t)((size_t)m_tiles * 32 * MT * MH * k * 2);  // (checked by the caller to fit)
    skn_launch(ctx, gemm_q4k_frag_kernel<MT, MH>, dim3(m_tiles * segs.n_tiles), dim3(256 * MH), kLds, afrag, sfrag, segs, isc, m, k, a_bytes);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

// ---- Q4_K path for wide weight matrices: a 256 x 128 tile, weights unpacked once for all its rows -------------
// The arithmetic of gemm_q4k_frag_kernel with its two costs divided differently.  A workgroup of eight wavefronts
// holds a 256 x 128 tile and walks k superblock by superblock.  Four consumers, one per SIMD, own 64 rows each --
// a 64 x 128 tile per wavefront: an activation fragment feeds four matrix instructions instead of two, so the
// activations a compute unit takes in per matrix instruction halve -- and four producers, their SIMD neighbours, own
// 32 columns each: a producer unpacks the fragments of its columns once for all 256 rows (a quarter of the vector
// instructions per matrix instruction of the other kernel) into LDS, two phases (a phase: a chunk of 64 elements,
// four k-steps) ahead of the consumers, three buffers, one bare barrier per phase; entering a superblock it leaves
// the min operands and the ratio by which the accumulators change their unit beside them.  The consumers load their
// activation fragments themselves (ring of eight k-steps), read the weight fragments one k-step ahead -- across the
// barrier too: what the next phase starts with was complete a phase ago -- and issue the matrix instructions; the
// change of unit between two superblocks is spread between the matrix instructions around it.  No split of k, so no
// exchange at the end.  (Timed in the kernel, the loop of one workgroup alone on the device takes as many core clocks
// as with all 224 -- nothing shared between compute units holds it -- but the core clock falls from 2.39 GHz to
// 1.8 - 1.9 GHz with all compute units at this work.)
constexpr int kTlStage = 4 * 4 * 1024;           // a phase: four k-steps x four column blocks x 1 KiB
constexpr int kTlAux = 128 * 32 + 128 * 4;       // a superblock's min operands (128 columns x (hi, lo) x 16 B) and ratios
constexpr int kTlLds = 3 * kTlStage + 2 * kTlAux + 128 * 4 + 256 * 4;

// One to three matrices per launch as in gemm_q4k_frag_kernel (tile0 counts 128-column tiles here); pair: a tile holds
// the same 64 columns of the gate and the up matrix -- producers 0 and 1 unpack the gate's, 2 and 3 the up's, so a
// consumer's column blocks 0, 1 and 2, 3 meet lane by lane in the store -- and stores silu(gate) * up into c[0].
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void gemm_q4k_tall_kernel(const u32x4* __restrict__ afrag, const u32x4* __restrict__ sfrag, const Q4kFragSegs segs,
                          const float* __restrict__ inv_scale, int m, int k, int m_tiles, uint32_t a_bytes) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const int me = wave & 3;  // consumer: its 64 rows; producer: its 32 columns
    const bool producer = wave >= 4;
    const int h = lane >> 5, r = lane & 31;
    const int nb = k >> 8, nch = k >> 6;
    const int mt = blockIdx.x % m_tiles, tn = blockIdx.x / m_tiles;  // (the row tiles of a column tile run side by side)
    const bool pair = segs.pair != 0;
    const int seg = pair ? 0 : (tn >= segs.tile0[2] ? 2 : (tn >= segs.tile0[1] ? 1 : 0));
    const int n = segs.n[seg];
    const int n0 = pair ? tn * 64 : (tn - segs.tile0[seg]) * 128;  // first column of the tile in its matrix (pair: in both)
    float* __restrict__ c = segs.c[seg];
    uint8_t* stage = lds;
    uint8_t* aux = lds + 3 * kTlStage;
    uint8_t* fin = aux + 2 * kTlAux;
    float* isc_lds = reinterpret_cast<float*>(fin + 128 * 4);  // the scales of the tile's 256 rows, for the store at the end
    if (tid < 256) isc_lds[tid] = inv_scale[mt * 256 + tid];
    auto barrier = [&]() __attribute__((always_inline)) { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
    using C0 = std::integral_constant<int, 0>;
    using C1 = std::integral_constant<int, 1>;
    using C2 = std::integral_constant<int, 2>;
    using C3 = std::integral_constant<int, 3>;
    // the three buffers in turn: phase p is multiplied from b_cur, phase p + 1 lies complete in b_nxt, phase p + 2 is
    // being written to b_nx2 (byte offsets, uniform)
    int b_cur = 0, b_nxt = kTlStage, b_nx2 = 2 * kTlStage;
    auto turn = [&]() __attribute__((always_inline)) {
        const int t = b_cur;
        b_cur = b_nxt, b_nxt = b_nx2, b_nx2 = t;
    };

    if (producer) {
        const uint8_t* w = segs.w[pair ? me >> 1 : seg];
        const __amdgpu_buffer_rsrc_t wrsrc = __builtin_amdgcn_make_buffer_rsrc((void*)w, 0, n * nb * 144, 0x00020000);  // (checked by the caller to fit)
        const int col = 32 * me + r;  // column of the tile
        const int wrow = min(n0 + (pair ? 32 * (me & 1) + r : col), n - 1) * nb * 144;
        // One set of registers for the header and the four nibble pieces; each is requested again, for the next
        // superblock, right after it is unpacked: four phases before its next use.
        u32x4 hd, q[4];
        auto load_piece = [&](int sb, int cc) __attribute__((always_inline)) {
            sb = min(sb, nb - 1);  // (past the end: a repeat, unused)
            q[cc] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, wrow + 16 * h, sb * 144 + 16 + 32 * cc, 0));
        };
        auto load_header = [&](int sb) __attribute__((always_inline)) {
            sb = min(sb, nb - 1);
            hd = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, wrow, sb * 144, 0));
        };
        uint32_t sc4[2], mn4[2];
        float sc_unit = 1.f, cs = 1.f;
        auto byte_f = [](uint32_t word, int b) { return (float)((word >> (8 * b)) & 0xFFu); };
        // header of the superblock in hd -> scales, mins, units; its ratio and min operands into aux[sb & 1]
        auto enter = [&](int sb) __attribute__((always_inline)) {
            uint8_t* ax = aux + (sb & 1) * kTlAux;
            // (the header is taken up here and no earlier: without this the compiler computes on it, and waits for
            // it, phases before)
            asm volatile("" : "+v"(hd));
            const uint32_t dw0 = hd[0], s0 = hd[1], s1 = hd[2], s2 = hd[3];
            const half2_t dd = __builtin_bit_cast(half2_t, dw0);
            const float d = (float)dd.x, dmin = (float)dd.y;
            const bool live = d != 0.f;  // (a zero d: the products are zeroed)
            sc4[0] = live ? s0 & 0x3F3F3F3Fu : 0u;
            sc4[1] = live ? (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u) : 0u;
            mn4[0] = s1 & 0x3F3F3F3Fu;
            mn4[1] = ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u);
            // (units, power pw and saturation as in gemm_q4k_frag_kernel)
            const int e_d = (int)((__float_as_uint(d) >> 23) & 0xFFu), e_m = (int)((__float_as_uint(dmin) >> 23) & 0xFFu);
            const int pw = live ? min(max(e_m - e_d - 10, 0), 10) : 0;
            sc_unit = __uint_as_float((uint32_t)(127 + 10 - pw) << 23);
            const float cs_new = live ? d * __uint_as_float((uint32_t)(127 + 14 + pw) << 23)
                                      : (dmin != 0.f ? fabsf(dmin) * 512.0f : cs);
            const float inv = 1.0f / cs_new, ratio = cs * inv;
            const float min_unit = fminf(fmaxf(-dmin * inv * 4096.0f, -1023.f), 1023.f);
            cs = cs_new;
            if (h == 0) {
                half8_t vh, vl;
#pragma unroll
                for (int x = 0; x < 8; x++) {
                    _Float16 a, b;
                    skn_split_hilo(min_unit * byte_f(mn4[x >> 2], x & 3), a, b);
                    vh[x] = a, vl[x] = b;
                }
                *reinterpret_cast<half8_t*>(ax + col * 32) = vh;
                *reinterpret_cast<half8_t*>(ax + col * 32 + 16) = vl;
                *reinterpret_cast<float*>(ax + 128 * 32 + col * 4) = ratio;
            }
        };
        // chunk cc of the superblock in q -> four k-steps of this producer's column block into the buffer at `buf`
        auto unpack = [&](auto cc_const, int buf) __attribute__((always_inline)) {
            constexpr int cc = decltype(cc_const)::value;
            uint8_t* dst = stage + buf + me * 1024 + lane * 16;
            asm volatile("" : "+v"(q[cc]));  // (as for the header)
            const float fl = byte_f(sc4[cc >> 1], 2 * (cc & 1)) * sc_unit;
            const float fh = byte_f(sc4[cc >> 1], 2 * (cc & 1) + 1) * (sc_unit * 0.0625f);
            const half2_t mul_lo = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_pkrtz(fl, fl));  // (six bits times a power of two: exact)
            const half2_t mul_hi = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_pkrtz(fh, fh));
#pragma unroll
            for (int s4 = 0; s4 < 4; s4++) {
                const uint32_t qq = q[cc][s4], q8 = qq >> 8;
                const uint32_t l02 = qq & 0x000F000Fu, h02 = qq & 0x00F000F0u;
                const uint32_t l13 = q8 & 0x000F000Fu, h13 = q8 & 0x00F000F0u;
                u32x4 o;
                o.x = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, l02) * mul_lo);
                o.y = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, h02) * mul_hi);
                o.z = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, l13) * mul_lo);
                o.w = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, h13) * mul_hi);
                *reinterpret_cast<u32x4*>(dst + s4 * 4096) = o;
            }
        };
        // While the consumers multiply phase (sb, cc) the producer unpacks the phase two after it -- chunks 2 and 3 of
        // the superblock, then chunks 0 and 1 of the next, whose header it takes up with chunk 0 -- and requests the
        // same piece of the superblock after that.  (After the last superblock it unpacks a repeat into buffers that
        // nobody reads any more -- no branch, so that the requests are not moved down into one -- and keeps the unit.)
        auto phase = [&](int sb, auto cc_const) __attribute__((always_inline)) {
            constexpr int cc = decltype(cc_const)::value;
            if (cc == 0) {
                unpack(C2{}, b_nx2);
                load_piece(sb + 1, 2);
            }
            if (cc == 1) {
                unpack(C3{}, b_nx2);
                load_piece(sb + 1, 3);
            }
            if (cc == 2) {
                const float keep = cs;
                enter(sb + 1);
                if (sb + 1 >= nb) cs = keep;
                unpack(C0{}, b_nx2);
                load_header(sb + 2);
                load_piece(sb + 2, 0);
            }
            if (cc == 3) {
                unpack(C1{}, b_nx2);
                load_piece(sb + 2, 1);
            }
            barrier();
            turn();
        };
        load_header(0);
#pragma unroll
        for (int x = 0; x < 4; x++) load_piece(0, x);
        enter(0);
        unpack(C0{}, b_cur);
        unpack(C1{}, b_nxt);
        load_header(1);
        load_piece(1, 0);
        load_piece(1, 1);
        barrier();
        for (int sb = 0; sb < nb; sb++) {
            phase(sb, C0{});
            phase(sb, C1{});
            phase(sb, C2{});
            phase(sb, C3{});
        }
        // the unit the accumulators ended in
        if (h == 0) *reinterpret_cast<float*>(fin + col * 4) = cs;
        barrier();
    } else {
        constexpr int MT = 2;
        const __amdgpu_buffer_rsrc_t arsrc = __builtin_amdgcn_make_buffer_rsrc((void*)afrag, 0, (int)a_bytes, 0x00020000);
        const int mb0 = mt * 8 + me * MT;  // first row block of this consumer
        uint32_t abase[MT];
#pragma unroll
        for (int i = 0; i < MT; i++) abase[i] = (uint32_t)(mb0 + i) * (uint32_t)nch * 4096u;
        u32x4 a[8][MT];  // ring of eight k-steps, seven ahead
        auto afetch = [&](int step, int slot) __attribute__((always_inline)) {  // step: absolute, 16 per superblock
            step = min(step, 16 * nb - 1);  // (past the end: the last step again, unused)
#pragma unroll
            for (int i = 0; i < MT; i++)
                a[slot][i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(arsrc, lane * 16, (int)(abase[i] + (uint32_t)step * 1024u), 0));
        };
        float16_t acc[MT][4];
#pragma unroll
        for (int i = 0; i < MT; i++)
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int x = 0; x < 16; x++) acc[i][j][x] = 0.f;
        u32x4 sf[MT];
        half8_t fb[2][4];  // the weight fragments of a k-step, read while the step before it is multiplied; step 0 of a phase in fb[0]
        float ratio[4] = {1.f, 1.f, 1.f, 1.f};  // of the superblock being entered, by column block
        // tile t = 4 i + j changes its unit: half `part` of its sixteen registers
        auto rescale = [&](int t, int part) __attribute__((always_inline)) {
#pragma unroll
            for (int x = 0; x < 8; x++) acc[t >> 2][t & 3][8 * part + x] *= ratio[t & 3];
        };
        auto fence = [&]() __attribute__((always_inline)) { __builtin_amdgcn_sched_barrier(0); };
        auto phase = [&](int sb, auto cc_const) __attribute__((always_inline)) {
            constexpr int cc = decltype(cc_const)::value;
            const uint8_t* ax = aux + (sb & 1) * kTlAux;
            const uint8_t* axn = aux + ((sb + 1) & 1) * kTlAux;
            if (cc == 0) {  // (the sub-block sums of the rows: needed three phases on)
#pragma unroll
                for (int i = 0; i < MT; i++) sf[i] = sfrag[((size_t)(mb0 + i) * nb + sb) * 64 + lane];
            }
            const uint8_t* src = stage + b_cur + lane * 16;
            const uint8_t* srcn = stage + b_nxt + lane * 16;
            half8_t vh[4], vl[4];
            float rnext[4];
            if (cc == 3) {  // (the ratios of the next superblock, left by the producers a phase ago: used at the end of this phase)
#pragma unroll
                for (int j = 0; j < 4; j++) rnext[j] = *reinterpret_cast<const float*>(axn + 128 * 32 + (j * 32 + r) * 4);
            }
#pragma unroll
            for (int s4 = 0; s4 < 4; s4++) {
                const int step = 4 * cc + s4, slot = step & 7;
                if (s4 < 3) {
#pragma unroll
                    for (int j = 0; j < 4; j++) fb[(s4 + 1) & 1][j] = *reinterpret_cast<const half8_t*>(src + (s4 + 1) * 4096 + j * 1024);
                } else if (cc < 3) {  // the next phase's first step: complete since the barrier before this phase
#pragma unroll
                    for (int j = 0; j < 4; j++) fb[0][j] = *reinterpret_cast<const half8_t*>(srcn + j * 1024);
                } else {
#pragma unroll
                    for (int j = 0; j < 4; j++) vh[j] = *reinterpret_cast<const half8_t*>(ax + (j * 32 + r) * 32);
                }
                fence();
                if (cc == 0 && s4 == 0) {
                    // the superblock's first step: tiles 3 .. 7 change their unit between its matrix instructions
                    // (tiles 0 .. 2 did before the barrier)
#pragma unroll
                    for (int t = 0; t < 8; t++) {
                        acc[t >> 2][t & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a[slot][t >> 2]), fb[0][t & 3],
                                                                                    acc[t >> 2][t & 3], 0, 0, 0);
                        fence();
                        if (t < 4) rescale(3 + (t >> 1), t & 1);
                        if (t >= 4 && t < 7) rescale(t + 1, 0), rescale(t + 1, 1);
                        fence();
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < MT; i++) {
                        const half8_t fa = __builtin_bit_cast(half8_t, a[slot][i]);
#pragma unroll
                        for (int j = 0; j < 4; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa, fb[s4 & 1][j], acc[i][j], 0, 0, 0);
                    }
                }
                afetch(16 * sb + step + 7, (step + 7) & 7);
                fence();
            }
            if (cc == 3) {
                // The "- dmin * m" term of the superblock (the two products of a tile eight instructions apart), and
                // under it the reads for what follows: the low parts, then the next phase's first step.
#pragma unroll
                for (int j = 0; j < 4; j++) vl[j] = *reinterpret_cast<const half8_t*>(ax + (j * 32 + r) * 32 + 16);
                fence();
#pragma unroll
                for (int i = 0; i < MT; i++)
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, sf[i]), vh[j], acc[i][j], 0, 0, 0);
                fence();
#pragma unroll
                for (int j = 0; j < 4; j++) fb[0][j] = *reinterpret_cast<const half8_t*>(srcn + j * 1024);
#pragma unroll
                for (int j = 0; j < 4; j++) ratio[j] = sb + 1 < nb ? rnext[j] : 1.0f;  // (none after the last superblock)
                fence();
                // tiles 0 .. 2 change their unit between the last of these instructions
#pragma unroll
                for (int t = 0; t < 8; t++) {
                    acc[t >> 2][t & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, sf[t >> 2]), vl[t & 3], acc[t >> 2][t & 3], 0, 0, 0);
                    fence();
                    if (t >= 2) rescale((t - 2) >> 1, t & 1);
                    fence();
                }
            }
            barrier();
            turn();
        };
#pragma unroll
        for (int s = 0; s < 7; s++) afetch(s, s);
        barrier();
#pragma unroll
        for (int j = 0; j < 4; j++) fb[0][j] = *reinterpret_cast<const half8_t*>(stage + b_cur + lane * 16 + j * 1024);
        for (int sb = 0; sb < nb; sb++) {
            phase(sb, C0{});
            phase(sb, C1{});
            phase(sb, C2{});
            phase(sb, C3{});
        }
        barrier();
#pragma unroll
        for (int i = 0; i < MT; i++) {
            float sc[16];
#pragma unroll
            for (int x = 0; x < 16; x++) sc[x] = isc_lds[(me * MT + i) * 32 + 8 * (x >> 2) + 4 * h + (x & 3)];
            if (pair) {
#pragma unroll
                for (int jj = 0; jj < 2; jj++) {
                    const float ug = *reinterpret_cast<const float*>(fin + (jj * 32 + r) * 4);
                    const float uu = *reinterpret_cast<const float*>(fin + ((jj + 2) * 32 + r) * 4);
                    const int col = n0 + 32 * jj + r;
#pragma unroll
                    for (int x = 0; x < 16; x++) {
                        // register x of lane l: row 8 (x / 4) + 4 (l / 32) + x % 4 of the 32 x 32 tile
                        const int row = (mb0 + i) * 32 + 8 * (x >> 2) + 4 * h + (x & 3);
                        if (row < m && col < n) {
                            const float g = acc[i][jj][x] * ug * sc[x], u = acc[i][jj + 2][x] * uu * sc[x];
                            c[(size_t)row * n + col] = g / (1.0f + expf(-g)) * u;  // silu(gate) * up
                        }
                    }
                }
                continue;
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float unit = *reinterpret_cast<const float*>(fin + (j * 32 + r) * 4);
#pragma unroll
                for (int x = 0; x < 16; x++) acc[i][j][x] *= unit;
                store_tile_scaled(acc[i][j], c, n, (mb0 + i) * 32, n0 + 32 * j, m, n, sc, lane, segs.accumulate[seg] != 0);
            }
        }
    }
}

// ---- general path: activations x (hi + lo * 2^-11) weights, both operands loaded in fragment order ---------
// Workgroup of four wavefronts, one per SIMD, tile (32 MT) x 64.  The tile is not divided spatially: wavefront
// kq computes all of it over a quarter of k (k is a multiple of 64, so the k-steps divide evenly) and the four
// partial tiles are added through LDS at the end, so no operand is loaded twice inside a workgroup.  Per k-step
// a wavefront loads MT activation fragments and four weight fragments (two column tiles, hi and lo) -- coalesced
// 1 KiB loads straight into the registers the matrix instructions read, D steps ahead -- and issues 4 MT matrix
// instructions.  Consecutive workgroups on an XCD (blockIdx / 8) are the row tiles of one column tile, so a
// weight fragment comes from memory once and from that XCD's L2 for the other row tiles.
template <int MT, int D>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void gemm_hilo_frag_kernel(const u32x4* __restrict__ afrag, const u32x4* __restrict__ bfrag,
                           const float* __restrict__ inv_scale, float* __restrict__ c, int m, int n, int steps,
                           int m_tiles, int n_tiles, int accumulate) {
    extern __shared__ __align__(16) float red[];  // 2 MT tiles x 3 copies x 1024 floats
    const int lane = threadIdx.x & 63, kq = threadIdx.x >> 6;
    const int slot_in_xcd = blockIdx.x >> 3;
    const int mt = slot_in_xcd % m_tiles, tn = (slot_in_xcd / m_tiles) * 8 + (blockIdx.x & 7);
    if (tn >= n_tiles) return;
    const int U = steps >> 2, t0 = kq * U;  // this wavefront's k-steps [t0, t0 + U)
    const u32x4* ap = afrag + ((size_t)mt * MT * steps + t0) * 64 + lane;   // + i * steps * 64 per row block
    const u32x4* bp = bfrag + ((size_t)tn * 2 * steps + t0) * 128 + lane;   // + j * steps * 128 per column block

    u32x4 ra[D][MT], rb[D][2][2];
    auto fetch = [&](int u, int slot) __attribute__((always_inline)) {
        u = min(u, U - 1);
#pragma unroll
        for (int i = 0; i < MT; i++) ra[slot][i] = ap[((size_t)i * steps + u) * 64];
#pragma unroll
        for (int j = 0; j < 2; j++) {
            rb[slot][j][0] = bp[((size_t)j * steps + u) * 128];
            rb[slot][j][1] = bp[((size_t)j * steps + u) * 128 + 64];
        }
    };
    float16_t acc[MT][2], accl[MT][2];
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int x = 0; x < 16; x++) acc[i][j][x] = accl[i][j][x] = 0.f;
    auto mac = [&](int slot) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < MT; i++) {
            const half8_t fa = __builtin_bit_cast(half8_t, ra[slot][i]);
#pragma unroll
            for (int j = 0; j < 2; j++) {
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa, __builtin_bit_cast(half8_t, rb[slot][j][0]), acc[i][j], 0, 0, 0);
                accl[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa, __builtin_bit_cast(half8_t, rb[slot][j][1]), accl[i][j], 0, 0, 0);
            }
        }
    };

    // Ring of D slots, D - 1 steps ahead: while the matrix instructions of step u run, the slot of step u - 1 --
    // whose registers are all free by then -- is refilled, one load after every second matrix instruction.
    // (Measured: the depth does not matter from 3 to 6 -- the loop is bound by operand delivery, 2 MiB per
    // compute unit and tile, not by its latency.)
#pragma unroll
    for (int x = 0; x < D - 1; x++) fetch(x, x);
    int u0 = 0;
    for (; u0 + D <= U; u0 += D) {
#pragma unroll
        for (int x = 0; x < D; x++) {
            fetch(u0 + x + D - 1, (x + D - 1) % D);  // (past the end: a repeat of the last step, unused)
            mac(x);
#pragma unroll
            for (int g = 0; g < MT + 4; g++) {
                __builtin_amdgcn_sched_group_barrier(0x008, (4 * MT) / (MT + 4), 0);  // matrix instructions
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);                    // one load
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // the last U % D steps are already in slots 0 ..
#pragma unroll
    for (int x = 0; x < D - 1; x++)
        if (u0 + x < U) mac(x);

    // hi + lo * 2^-11, then the four partial tiles: tile t = 2 i + j belongs to wavefront t % 4, the other three
    // hand theirs over
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
#pragma unroll
            for (int x = 0; x < 16; x++) acc[i][j][x] += accl[i][j][x] * 0x1p-11f;
            const int t = 2 * i + j, owner = t & 3;
            if (kq != owner) {
                float* dst = red + (t * 3 + ((kq - owner + 4) & 3) - 1) * 1024 + lane;
#pragma unroll
                for (int x = 0; x < 16; x++) dst[64 * x] = acc[i][j][x];
            }
        }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int t = 2 * i + j;
            if (kq == (t & 3)) {
                float16_t sum = acc[i][j];
#pragma unroll
                for (int o = 0; o < 3; o++)
#pragma unroll
                    for (int x = 0; x < 16; x++) sum[x] += red[(t * 3 + o) * 1024 + 64 * x + lane];
                store_tile(sum, c, n, (mt * MT + i) * 32, tn * kBN + 32 * j, m, n, inv_scale, lane, accumulate != 0);
            }
        }
}

template <int MT, int D>
int launch_hilo_gemm(skn_ctx* ctx, const u32x4* afrag, const u32x4* bfrag, const float* isc, float* c, int m, int n, int k,
                     int accumulate = 0) {
    constexpr int kLds = 2 * MT * 3 * 4096;
    const int m_tiles = (m + 32 * MT - 1) / (32 * MT), n_tiles = (n + kBN - 1) / kBN;
    const unsigned grid = (unsigned)(((n_tiles + 7) / 8) * 8 * m_tiles);
    skn_launch(ctx, gemm_hilo_frag_kernel<MT, D>, dim3(grid), dim3(256), kLds, afrag, bfrag, isc, c, m, n, k >> 4, m_tiles, n_tiles,
               accumulate);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

// row blocks per tile of the general path: 32 MT rows
inline int hilo_mt(int m) { return m <= 32 ? 1 : (m <= 64 ? 2 : 4); }

int launch_hilo_gemm_mt(skn_ctx* ctx, int mt, const u32x4* afrag, const u32x4* bfrag, const float* isc, float* c, int m, int n,
                        int k, int accumulate) {
    if (mt == 1) return launch_hilo_gemm<1, 4>(ctx, afrag, bfrag, isc, c, m, n, k, accumulate);
    if (mt == 2) return launch_hilo_gemm<2, 4>(ctx, afrag, bfrag, isc, c, m, n, k, accumulate);
    return launch_hilo_gemm<4, 4>(ctx, afrag, bfrag, isc, c, m, n, k, accumulate);
}

// ---- Q6_K path: weights unpacked in the kernel, two matrix instructions per k-step -----------------------
// w[n, 256 b + e] = d * sc_g * (q - 32) with q in 0..63, sc_g an int8 (one per sixteen elements), d fp16.  The integer
// sc_g (q - 32) needs thirteen bits, two more than an fp16 operand holds, so the scale is split, sc = 16 s1 + s0 with
// s0 in 0..15 and s1 in -8..7: (q - 32) s1 and (q - 32) s0 / 16 are exact fp16 numbers, each goes through the matrix
// core into the same accumulator, which then holds sum a sc (q - 32) / 16 of the superblock; at its end 16 d times
// that is added to the tile's running total and the accumulator starts again from zero (the first matrix instruction
// of a superblock takes no addend).  A quant is put together in place as the fp16 number 1024 + q (0x6400 | q: the
// low four bits masked out of ql, the two high bits out of qh shifted beside them), a pair per register, and one
// packed fused multiply-add per part, (1024 + q) s - 1056 s, makes the operand: the product is exact inside the
// instruction and 1056 s = 33 s 2^5 is an fp16 number, so nothing is rounded before the fp32 accumulation.
// Workgroup of four wavefronts, one per SIMD, tile (32 MT) x 64 as in the general path below: wavefront kq takes
// superblocks kq, kq + 4, ... of all the tile and the four partial tiles are added through LDS at the end.  The
// activations come in the fragment order of the Q4_K path; the element order inside a k-step -- 4 dw + {0, 2},
// 32 + 4 dw + {0, 2}, 4 dw + {1, 3}, 32 + 4 dw + {1, 3} with dw = 4 h + s in a chunk of 64 -- is the one Q6_K's own
// layout hands out: inside a half of 128 elements, element 32 Q + l has its low bits in nibble Q / 2 of byte
// 32 (Q % 2) + l of ql and its high bits at 2 Q of byte l of qh, so chunk c of the superblock (quarters 2 (c % 2) and
// 2 (c % 2) + 1 of half c / 2) takes dword s of three sixteen-byte pieces per lane -- ql + 64 (c / 2) + 16 h, the same
// + 32, qh + 32 (c / 2) + 16 h -- shifted right by 4 (c % 2).  Each lane reads the pieces of its own weight row (32
// rows per request, 210 bytes per superblock, no alignment beyond two bytes) straight into registers, half a
// superblock ahead; nothing but the final exchange passes through LDS and the loop has no barrier.
struct Q6kHalf {
    u32x4 qa[2], qb[2], qh[2];  // per 32-column block: ql + 16 h, ql + 32 + 16 h, qh + 16 h of the half
};

template <int MT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void gemm_q6k_frag_kernel(const u32x4* __restrict__ afrag, const uint8_t* __restrict__ w, const float* __restrict__ inv_scale,
                          float* __restrict__ c, int m, int n, int k, int m_tiles, int n_tiles, int accumulate,
                          uint32_t a_bytes, uint32_t w_bytes, int xcd_rows) {
    extern __shared__ __align__(16) float red[];  // 2 MT tiles x 3 copies x 1024 floats
    const int lane = threadIdx.x & 63;
    const int kq = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int h = lane >> 5, r = lane & 31;
    // Workgroup -> tile.  The packed weights of a tile are small (53 KiB per 64 columns at k = 4096) beside the
    // activations of its rows (1 MiB per 128 rows), so with up to eight row tiles an XCD (blockIdx % 8) keeps to one
    // row tile, whose activations then stay in its L2 while the column tiles stream through.
    int mt, tn;
    if (xcd_rows) {
        const int xcd = blockIdx.x & 7, per = 8 / m_tiles;
        mt = xcd % m_tiles;
        tn = (blockIdx.x >> 3) * per + xcd / m_tiles;
    } else {
        const int slot_in_xcd = blockIdx.x >> 3;
        mt = slot_in_xcd % m_tiles;
        tn = (slot_in_xcd / m_tiles) * 8 + (blockIdx.x & 7);
    }
    if (tn >= n_tiles) return;
    const int nb = k >> 8, nch = k >> 6;
    // The weights are read with buffer loads too: the lane's byte offset (its weight row, its sixteen-byte half) plus
    // a scalar one (superblock, piece).  A piece of an odd superblock starts at an address that is only a multiple
    // of two.
    const __amdgpu_buffer_rsrc_t wrsrc = __builtin_amdgcn_make_buffer_rsrc((void*)w, 0, (int)w_bytes, 0x00020000);
    int wrow[2];
#pragma unroll
    for (int j = 0; j < 2; j++) wrow[j] = min(tn * kBN + 32 * j + r, n - 1) * nb * 210 + 16 * h;

    const __amdgpu_buffer_rsrc_t arsrc = __builtin_amdgcn_make_buffer_rsrc((void*)afrag, 0, (int)a_bytes, 0x00020000);
    uint32_t abase[MT];
#pragma unroll
    for (int i = 0; i < MT; i++) abase[i] = (uint32_t)(mt * MT + i) * (uint32_t)nch * 4096u;
    constexpr int RING = 4;  // ring of k-steps, RING - 1 ahead (eight deep: the same time)
    u32x4 a[RING][MT];
    auto afetch = [&](int step, int slot) __attribute__((always_inline)) {  // step: 16 per superblock, absolute
#pragma unroll
        for (int i = 0; i < MT; i++)
            a[slot][i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(arsrc, lane * 16, (int)(abase[i] + (uint32_t)step * 1024u), 0));
    };
    auto wload = [&](int j, int off) __attribute__((always_inline)) {
        return __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, wrow[j], off, 0));
    };
    auto load_half = [&](int sb, int hf, Q6kHalf& H) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            H.qa[j] = wload(j, sb * 210 + 64 * hf);
            H.qb[j] = wload(j, sb * 210 + 64 * hf + 32);
            H.qh[j] = wload(j, sb * 210 + 128 + 32 * hf);
        }
    };
    // the sixteen scales of the superblock (both halves of the lanes read all of them: the lane's own sixteen-byte
    // offset is taken back out) and its d, per column block
    u32x4 scl[2], scl_n[2];
    uint32_t dh[2], dh_n[2];
    auto load_head = [&](int sb, u32x4 (&sc_out)[2], uint32_t (&d_out)[2]) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            sc_out[j] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, wrow[j] - 16 * h, sb * 210 + 192, 0));
            d_out[j] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(wrsrc, wrow[j] - 16 * h, sb * 210 + 208, 0);
        }
    };

    float16_t acc[MT][2], total[MT][2];
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int x = 0; x < 16; x++) total[i][j][x] = 0.f;

    Q6kHalf H0, H1;
    if (kq < nb) {
        load_head(kq, scl_n, dh_n);
        load_half(kq, 0, H0);
#pragma unroll
        for (int s = 0; s < RING - 1; s++) afetch(16 * kq + s, s);
    }
    for (int sb = kq; sb < nb; sb += 4) {
        const int sb_next = min(sb + 4, nb - 1);  // (past the end: a repeat of the last superblock, unused)
        float dsc[2];
#pragma unroll
        for (int j = 0; j < 2; j++) {
            scl[j] = scl_n[j];
            dh[j] = dh_n[j];
            dsc[j] = (float)__builtin_bit_cast(_Float16, (uint16_t)dh[j]) * 16.0f;
        }
        // one chunk of 64 elements = four k-steps; cc = 0..3, its half is cc / 2
        auto chunk = [&](auto cc_const, const Q6kHalf& H) __attribute__((always_inline)) {
            constexpr int cc = decltype(cc_const)::value;
            constexpr int par = cc & 1;
            half2_t s0v[2][2], c0v[2][2], s1v[2][2], c1v[2][2];  // [column block][low 32 / high 32 of the chunk]
            u32x4 qa[2], qb[2], qh[2];
#pragma unroll
            for (int j = 0; j < 2; j++) {
                qa[j] = par ? H.qa[j] >> 4u : H.qa[j];
                qb[j] = par ? H.qb[j] >> 4u : H.qb[j];
                qh[j] = par ? H.qh[j] >> 4u : H.qh[j];
                const uint32_t dw = scl[j][cc];  // scales 4 cc .. 4 cc + 3: the lane's groups are bytes h and 2 + h
#pragma unroll
                for (int g = 0; g < 2; g++) {
                    const int sc = __builtin_amdgcn_sbfe((int)dw, (unsigned)(8 * h + 16 * g), 8u);
                    const float f0 = (float)(sc & 15) * 0.0625f, f1 = (float)(sc >> 4);
                    s0v[j][g] = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_pkrtz(f0, f0));  // (four bits and a power of two: exact)
                    s1v[j][g] = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_pkrtz(f1, f1));
                    c0v[j][g] = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_pkrtz(-1056.0f * f0, -1056.0f * f0));
                    c1v[j][g] = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_pkrtz(-1056.0f * f1, -1056.0f * f1));
                }
            }
#pragma unroll
            for (int s = 0; s < 4; s++) {
                half8_t f0[2], f1[2];
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const uint32_t x = qa[j][s], y = qb[j][s], z = qh[j][s];
                    const uint32_t x8 = x >> 8, y8 = y >> 8, z8 = z >> 8;
                    const half2_t t[4] = {
                        __builtin_bit_cast(half2_t, ((z & 0x00030003u) << 4) | ((x & 0x000F000Fu) | 0x64006400u)),
                        __builtin_bit_cast(half2_t, ((z & 0x000C000Cu) << 2) | ((y & 0x000F000Fu) | 0x64006400u)),
                        __builtin_bit_cast(half2_t, ((z8 & 0x00030003u) << 4) | ((x8 & 0x000F000Fu) | 0x64006400u)),
                        __builtin_bit_cast(half2_t, ((z8 & 0x000C000Cu) << 2) | ((y8 & 0x000F000Fu) | 0x64006400u))};
                    u32x4 o0, o1;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        o0[e] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(t[e], s0v[j][e & 1], c0v[j][e & 1]));
                        o1[e] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(t[e], s1v[j][e & 1], c1v[j][e & 1]));
                    }
                    f0[j] = __builtin_bit_cast(half8_t, o0);
                    f1[j] = __builtin_bit_cast(half8_t, o1);
                }
                const int step = 4 * cc + s, slot = step & (RING - 1);
                // (the two matrix instructions of a tile are kept eight apart; the first of a superblock takes no addend)
                const float16_t zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int i = 0; i < MT; i++) {
                    const half8_t fa = __builtin_bit_cast(half8_t, a[slot][i]);
#pragma unroll
                    for (int j = 0; j < 2; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa, f1[j], step == 0 ? zero : acc[i][j], 0, 0, 0);
                }
#pragma unroll
                for (int i = 0; i < MT; i++) {
                    const half8_t fa = __builtin_bit_cast(half8_t, a[slot][i]);
#pragma unroll
                    for (int j = 0; j < 2; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa, f0[j], acc[i][j], 0, 0, 0);
                }
                // the slot of step - 1 is free: refill it RING - 1 steps ahead
                const int ahead = step + RING - 1;
                afetch(ahead < 16 ? 16 * sb + ahead : 16 * sb_next + ahead - 16, ahead & (RING - 1));
            }
        };
        load_half(sb, 1, H1);
        chunk(std::integral_constant<int, 0>{}, H0);
        chunk(std::integral_constant<int, 1>{}, H0);
        load_head(sb_next, scl_n, dh_n);
        load_half(sb_next, 0, H0);
        chunk(std::integral_constant<int, 2>{}, H1);
        chunk(std::integral_constant<int, 3>{}, H1);
        // the superblock's sum, in units of 16 d, joins the total
#pragma unroll
        for (int i = 0; i < MT; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int x = 0; x < 16; x++) total[i][j][x] = fmaf(dsc[j], acc[i][j][x], total[i][j][x]);
    }

    // the four partial tiles: tile t = 2 i + j belongs to wavefront t % 4, the other three hand theirs over
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int t = 2 * i + j, owner = t & 3;
            if (kq != owner) {
                float* dst = red + (t * 3 + ((kq - owner + 4) & 3) - 1) * 1024 + lane;
#pragma unroll
                for (int x = 0; x < 16; x++) dst[64 * x] = total[i][j][x];
            }
        }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int t = 2 * i + j;
            if (kq == (t & 3)) {
                float16_t sum = total[i][j];
#pragma unroll
                for (int o = 0; o < 3; o++)
#pragma unroll
                    for (int x = 0; x < 16; x++) sum[x] += red[(t * 3 + o) * 1024 + 64 * x + lane];
                store_tile(sum, c, n, (mt * MT + i) * 32, tn * kBN + 32 * j, m, n, inv_scale, lane, accumulate != 0);
            }
        }
}

// The same arithmetic with the wavefronts specialised: a workgroup of eight, on every SIMD a producer that unpacks
// (the vector instructions above) and a consumer that loads activation fragments and issues the matrix instructions,
// so that the two kinds of instruction come from different wavefronts and overlap.  Pair kq takes superblocks kq,
// kq + 4, ...; a phase is a chunk of 64 elements (four k-steps, sixteen 1 KiB weight fragments per pair: two column
// blocks x two parts); the producer works one phase ahead into the other of two LDS buffers, one bare barrier per
// phase.  The consumer keeps one set of accumulators in units of 16 d of the latest superblock whose d is not zero,
// rescaled on entering a superblock by the ratio the producer leaves beside the fragments (gemm_q4k_frag_kernel's
// scheme), so that it needs no running total.
constexpr int kQ6Stage = 4 * 4 * 1024;         // a phase of one pair: four k-steps x (two column blocks x two parts) x 1 KiB
constexpr int kQ6Aux = 2 * 256 + 256;          // per pair: the ratios of two superblocks in turn, then the last unit
constexpr int kQ6PcLds = 4 * 2 * kQ6Stage + 4 * kQ6Aux;

__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void gemm_q6k_pc_kernel(const u32x4* __restrict__ afrag, const uint8_t* __restrict__ w, const float* __restrict__ inv_scale,
                        float* __restrict__ c, int m, int n, int k, int m_tiles, int n_tiles, int accumulate,
                        uint32_t a_bytes, uint32_t w_bytes) {
    constexpr int MT = 4;
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const int kq = wave & 3;
    const bool producer = wave >= 4;
    const int h = lane >> 5, r = lane & 31;
    const int xcd = blockIdx.x & 7, per = 8 / m_tiles;  // (an XCD keeps to one row tile, as above; m_tiles divides 8)
    const int mt = xcd % m_tiles, tn = (blockIdx.x >> 3) * per + xcd / m_tiles;
    if (tn >= n_tiles) return;
    const int nb = k >> 8, nch = k >> 6, nsb = (nb + 3) >> 2;  // nsb: superblocks of the busiest pair
    uint8_t* stage = lds + kq * 2 * kQ6Stage;
    uint8_t* aux = lds + 4 * 2 * kQ6Stage + kq * kQ6Aux;
    auto barrier = [&]() __attribute__((always_inline)) { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
    using C0 = std::integral_constant<int, 0>;
    using C1 = std::integral_constant<int, 1>;
    using C2 = std::integral_constant<int, 2>;
    using C3 = std::integral_constant<int, 3>;
    float* red = reinterpret_cast<float*>(lds);  // (for the end, when the stage buffers are free: 2 MT x 3 x 4 KiB of them)

    if (producer) {
        const __amdgpu_buffer_rsrc_t wrsrc = __builtin_amdgcn_make_buffer_rsrc((void*)w, 0, (int)w_bytes, 0x00020000);
        int wrow[2];
#pragma unroll
        for (int j = 0; j < 2; j++) wrow[j] = min(tn * kBN + 32 * j + r, n - 1) * nb * 210 + 16 * h;
        auto wload = [&](int j, int off) __attribute__((always_inline)) {
            return __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, wrow[j], off, 0));
        };
        auto load_half = [&](int sb, int hf, Q6kHalf& H) __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < 2; j++) {
                H.qa[j] = wload(j, sb * 210 + 64 * hf);
                H.qb[j] = wload(j, sb * 210 + 64 * hf + 32);
                H.qh[j] = wload(j, sb * 210 + 128 + 32 * hf);
            }
        };
        u32x4 scl[2], scl_n[2];
        uint32_t dh[2], dh_n[2];
        auto load_head = [&](int sb, u32x4 (&sc_out)[2], uint32_t (&d_out)[2]) __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < 2; j++) {
                sc_out[j] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, wrow[j] - 16 * h, sb * 210 + 192, 0));
                d_out[j] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(wrsrc, wrow[j] - 16 * h, sb * 210 + 208, 0);
            }
        };
        Q6kHalf H0, H1;
        float cs[2] = {1.f, 1.f};
        bool live[2] = {true, true};
        // entering superblock i (pair-local): its head becomes current, its ratio goes to aux[i & 1]
        auto enter = [&](int i) __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < 2; j++) {
                scl[j] = scl_n[j], dh[j] = dh_n[j];
                const float d = (float)__builtin_bit_cast(_Float16, (uint16_t)dh[j]);
                live[j] = d != 0.f;  // (a zero d: the products are zeroed and the unit stays)
                const float cs_new = live[j] ? d * 16.0f : cs[j];
                const float ratio = cs[j] / cs_new;
                cs[j] = cs_new;
                if (h == 0) *reinterpret_cast<float*>(aux + (i & 1) * 256 + (j * 32 + r) * 4) = ratio;
            }
        };
        // chunk cc of the current superblock -> sixteen fragments into buffer `buf`
        auto unpack = [&](auto cc_const, const Q6kHalf& H, int buf) __attribute__((always_inline)) {
            constexpr int cc = decltype(cc_const)::value;
            constexpr int par = cc & 1;
            uint8_t* dst = stage + buf * kQ6Stage + lane * 16;
            half2_t s0v[2][2], c0v[2][2], s1v[2][2], c1v[2][2];  // [column block][low 32 / high 32 of the chunk]
            u32x4 qa[2], qb[2], qh[2];
#pragma unroll
            for (int j = 0; j < 2; j++) {
                qa[j] = par ? H.qa[j] >> 4u : H.qa[j];
                qb[j] = par ? H.qb[j] >> 4u : H.qb[j];
                qh[j] = par ? H.qh[j] >> 4u : H.qh[j];
                const uint32_t dw = scl[j][cc];  // scales 4 cc .. 4 cc + 3: the lane's groups are bytes h and 2 + h
#pragma unroll
                for (int g = 0; g < 2; g++) {
                    const int sc = live[j] ? __builtin_amdgcn_sbfe((int)dw, (unsigned)(8 * h + 16 * g), 8u) : 0;
                    const float f0 = (float)(sc & 15) * 0.0625f, f1 = (float)(sc >> 4);
                    s0v[j][g] = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_pkrtz(f0, f0));  // (four bits and a power of two: exact)
                    s1v[j][g] = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_pkrtz(f1, f1));
                    c0v[j][g] = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_pkrtz(-1056.0f * f0, -1056.0f * f0));
                    c1v[j][g] = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_pkrtz(-1056.0f * f1, -1056.0f * f1));
                }
            }
#pragma unroll
            for (int s4 = 0; s4 < 4; s4++)
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const uint32_t x = qa[j][s4], y = qb[j][s4], z = qh[j][s4];
                    const uint32_t x8 = x >> 8, y8 = y >> 8, z8 = z >> 8;
                    const half2_t t[4] = {
                        __builtin_bit_cast(half2_t, ((z & 0x00030003u) << 4) | ((x & 0x000F000Fu) | 0x64006400u)),
                        __builtin_bit_cast(half2_t, ((z & 0x000C000Cu) << 2) | ((y & 0x000F000Fu) | 0x64006400u)),
                        __builtin_bit_cast(half2_t, ((z8 & 0x00030003u) << 4) | ((x8 & 0x000F000Fu) | 0x64006400u)),
                        __builtin_bit_cast(half2_t, ((z8 & 0x000C000Cu) << 2) | ((y8 & 0x000F000Fu) | 0x64006400u))};
                    u32x4 o0, o1;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        o0[e] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(t[e], s0v[j][e & 1], c0v[j][e & 1]));
                        o1[e] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(t[e], s1v[j][e & 1], c1v[j][e & 1]));
                    }
                    *reinterpret_cast<u32x4*>(dst + ((s4 * 2 + j) * 2 + 0) * 1024) = o1;
                    *reinterpret_cast<u32x4*>(dst + ((s4 * 2 + j) * 2 + 1) * 1024) = o0;
                }
        };
        // While the consumers multiply phase (i, cc) the producer unpacks the phase after it.  Requests, two phases
        // before their use: head and first half of the next superblock with chunk 2, its second half with its chunk 0.
        auto phase = [&](int i, auto cc_const) __attribute__((always_inline)) {
            constexpr int cc = decltype(cc_const)::value;
            const int sb = 4 * i + kq;
            if (sb < nb) {
                const int sbn = min(sb + 4, nb - 1);  // (past the end: a repeat, unused)
                if (cc == 0) unpack(C1{}, H0, 1);
                if (cc == 1) {
                    load_head(sbn, scl_n, dh_n);
                    load_half(sbn, 0, H0);
                    unpack(C2{}, H1, 0);
                }
                if (cc == 2) unpack(C3{}, H1, 1);
                if (cc == 3 && sb + 4 < nb) {
                    enter(i + 1);
                    load_half(sb + 4, 1, H1);
                    unpack(C0{}, H0, 0);
                }
            }
            barrier();
        };
        if (kq < nb) {
            load_head(kq, scl_n, dh_n);
            load_half(kq, 0, H0);
            load_half(kq, 1, H1);
            enter(0);
            unpack(C0{}, H0, 0);
        }
        barrier();
        for (int i = 0; i < nsb; i++) {
            phase(i, C0{});
            phase(i, C1{});
            phase(i, C2{});
            phase(i, C3{});
        }
        if (h == 0) {
#pragma unroll
            for (int j = 0; j < 2; j++) *reinterpret_cast<float*>(aux + 512 + (j * 32 + r) * 4) = cs[j];
        }
        barrier();
        barrier();
    } else {
        const __amdgpu_buffer_rsrc_t arsrc = __builtin_amdgcn_make_buffer_rsrc((void*)afrag, 0, (int)a_bytes, 0x00020000);
        uint32_t abase[MT];
#pragma unroll
        for (int i = 0; i < MT; i++) abase[i] = (uint32_t)(mt * MT + i) * (uint32_t)nch * 4096u;
        u32x4 a[4][MT];  // ring of four k-steps, three ahead
        auto afetch = [&](int step, int slot) __attribute__((always_inline)) {  // step: 16 per superblock, absolute
#pragma unroll
            for (int i = 0; i < MT; i++)
                a[slot][i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(arsrc, lane * 16, (int)(abase[i] + (uint32_t)step * 1024u), 0));
        };
        float16_t acc[MT][2];
#pragma unroll
        for (int i = 0; i < MT; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int x = 0; x < 16; x++) acc[i][j][x] = 0.f;
        auto phase = [&](int i, auto cc_const) __attribute__((always_inline)) {
            constexpr int cc = decltype(cc_const)::value;
            const int sb = 4 * i + kq;
            if (sb < nb) {
                if (cc == 0) {
#pragma unroll
                    for (int j = 0; j < 2; j++) {
                        const float ratio = *reinterpret_cast<const float*>(aux + (i & 1) * 256 + (j * 32 + r) * 4);
#pragma unroll
                        for (int ii = 0; ii < MT; ii++)
#pragma unroll
                            for (int x = 0; x < 16; x++) acc[ii][j][x] *= ratio;
                    }
                }
                const uint8_t* src = stage + (cc & 1) * kQ6Stage + lane * 16;
                const int sbn = min(sb + 4, nb - 1);
                // (the weight fragments of step s + 1 are read from LDS before the matrix instructions of step s are issued)
                half8_t fb[2][2][2];  // [step parity][column block][part]
#pragma unroll
                for (int j = 0; j < 2; j++)
#pragma unroll
                    for (int pt = 0; pt < 2; pt++) fb[0][j][pt] = *reinterpret_cast<const half8_t*>(src + (j * 2 + pt) * 1024);
#pragma unroll
                for (int s4 = 0; s4 < 4; s4++) {
                    const int step = 4 * cc + s4, slot = step & 3;
                    if (s4 + 1 < 4) {
#pragma unroll
                        for (int j = 0; j < 2; j++)
#pragma unroll
                            for (int pt = 0; pt < 2; pt++)
                                fb[(s4 + 1) & 1][j][pt] = *reinterpret_cast<const half8_t*>(src + (((s4 + 1) * 2 + j) * 2 + pt) * 1024);
                    }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int pt = 0; pt < 2; pt++)
#pragma unroll
                        for (int ii = 0; ii < MT; ii++) {
                            const half8_t fa = __builtin_bit_cast(half8_t, a[slot][ii]);
#pragma unroll
                            for (int j = 0; j < 2; j++)
                                acc[ii][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa, fb[s4 & 1][j][pt], acc[ii][j], 0, 0, 0);
                        }
                    const int ahead = step + 3;
                    afetch(ahead < 16 ? 16 * sb + ahead : 16 * sbn + ahead - 16, ahead & 3);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            barrier();
        };
        if (kq < nb) {
#pragma unroll
            for (int s = 0; s < 3; s++) afetch(16 * kq + s, s);
        }
        barrier();
        for (int i = 0; i < nsb; i++) {
            phase(i, C0{});
            phase(i, C1{});
            phase(i, C2{});
            phase(i, C3{});
        }
        barrier();
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const float unit = *reinterpret_cast<const float*>(aux + 512 + (j * 32 + r) * 4);
#pragma unroll
            for (int ii = 0; ii < MT; ii++) {
#pragma unroll
                for (int x = 0; x < 16; x++) acc[ii][j][x] *= unit;
                const int t = 2 * ii + j, owner = t & 3;
                if (kq != owner) {
                    float* dst = red + (t * 3 + ((kq - owner + 4) & 3) - 1) * 1024 + lane;
#pragma unroll
                    for (int x = 0; x < 16; x++) dst[64 * x] = acc[ii][j][x];
                }
            }
        }
        barrier();
#pragma unroll
        for (int ii = 0; ii < MT; ii++)
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int t = 2 * ii + j;
                if (kq == (t & 3)) {
                    float16_t sum = acc[ii][j];
#pragma unroll
                    for (int o = 0; o < 3; o++)
#pragma unroll
                        for (int x = 0; x < 16; x++) sum[x] += red[(t * 3 + o) * 1024 + 64 * x + lane];
                    store_tile(sum, c, n, (mt * MT + ii) * 32, tn * kBN + 32 * j, m, n, inv_scale, lane, accumulate != 0);
                }
            }
    }
}

// The same for wide weight matrices in the form of gemm_q4k_tall_kernel: a 256 x 128 tile, k walked superblock by
// superblock by all eight wavefronts; four consumers own 64 rows each (a 64 x 128 tile per wavefront), four producers
// 32 columns each, whose blocks they unpack once for all 256 rows into LDS (per k-step and column block the two
// parts of the split scale as two fragments), two phases (chunks of 64 elements) ahead, three buffers, one bare
// barrier per phase.  The consumers take the two parts one after the other (the same activation fragment, eight
// matrix instructions each) and read the next half-step's four fragments from LDS, across the barrier too, while the
// current eight instructions run.  Accumulators in units of 16 d as in gemm_q6k_pc_kernel, the change of unit spread
// between the matrix instructions on both sides of a superblock's end.
constexpr int kQ6TlStage = 4 * 8 * 1024;          // a phase: four k-steps x (four column blocks x two parts) x 1 KiB
constexpr int kQ6TlLds = 3 * kQ6TlStage + 2 * 128 * 4 + 128 * 4 + 256 * 4;

__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void gemm_q6k_tall_kernel(const u32x4* __restrict__ afrag, const uint8_t* __restrict__ w, const float* __restrict__ inv_scale,
                          float* __restrict__ c, int m, int n, int k, int m_tiles, int accumulate, uint32_t a_bytes,
                          uint32_t w_bytes) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const int me = wave & 3;  // consumer: its 64 rows; producer: its 32 columns
    const bool producer = wave >= 4;
    const int h = lane >> 5, r = lane & 31;
    const int nb = k >> 8, nch = k >> 6;
    const int mt = blockIdx.x % m_tiles, tn = blockIdx.x / m_tiles;  // (the row tiles of a column tile run side by side)
    const int n0 = tn * 128;
    uint8_t* stage = lds;
    float* ratios = reinterpret_cast<float*>(lds + 3 * kQ6TlStage);  // [superblock parity][128 columns]
    float* fin = ratios + 2 * 128;                                   // the last unit of the 128 columns
    float* isc_lds = fin + 128;                                      // the scales of the tile's 256 rows
    if (tid < 256) isc_lds[tid] = inv_scale[mt * 256 + tid];
    auto barrier = [&]() __attribute__((always_inline)) { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
    using C0 = std::integral_constant<int, 0>;
    using C1 = std::integral_constant<int, 1>;
    using C2 = std::integral_constant<int, 2>;
    using C3 = std::integral_constant<int, 3>;
    // the three buffers in turn: phase p is multiplied from b_cur, phase p + 1 lies complete in b_nxt, phase p + 2 is
    // being written to b_nx2 (byte offsets, uniform)
    int b_cur = 0, b_nxt = kQ6TlStage, b_nx2 = 2 * kQ6TlStage;
    auto turn = [&]() __attribute__((always_inline)) {
        const int t = b_cur;
        b_cur = b_nxt, b_nxt = b_nx2, b_nx2 = t;
    };

    if (producer) {
        const __amdgpu_buffer_rsrc_t wrsrc = __builtin_amdgcn_make_buffer_rsrc((void*)w, 0, (int)w_bytes, 0x00020000);
        const int col = 32 * me + r;
        const int wrow = min(n0 + col, n - 1) * nb * 210;
        u32x4 qa[2], qb[2], qh[2];  // [half of the superblock]: ql + 16 h, ql + 32 + 16 h, qh + 16 h
        u32x4 scl, scl_n;
        uint32_t dh_n = 0;
        auto load_half = [&](int sb, int hf) __attribute__((always_inline)) {
            sb = min(sb, nb - 1);  // (past the end: a repeat, unused)
            qa[hf] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, wrow + 16 * h, sb * 210 + 64 * hf, 0));
            qb[hf] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, wrow + 16 * h, sb * 210 + 64 * hf + 32, 0));
            qh[hf] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, wrow + 16 * h, sb * 210 + 128 + 32 * hf, 0));
        };
        auto load_head = [&](int sb) __attribute__((always_inline)) {
            sb = min(sb, nb - 1);
            scl_n = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, wrow, sb * 210 + 192, 0));
            dh_n = (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(wrsrc, wrow, sb * 210 + 208, 0);
        };
        float cs = 1.f;
        bool live = true;
        // entering superblock sb: its head becomes current, its ratio goes to ratios[sb & 1]
        auto enter = [&](int sb) __attribute__((always_inline)) {
            asm volatile("" : "+v"(scl_n), "+v"(dh_n));  // (taken up here and no earlier)
            scl = scl_n;
            const float d = (float)__builtin_bit_cast(_Float16, (uint16_t)dh_n);
            live = d != 0.f;  // (a zero d: the products are zeroed and the unit stays)
            const float cs_new = live ? d * 16.0f : cs;
            const float ratio = cs / cs_new;
            cs = cs_new;
            if (h == 0) ratios[(sb & 1) * 128 + col] = ratio;
        };
        // chunk cc of the current superblock -> four k-steps x two parts of this producer's column block into the buffer at `buf`
        auto unpack = [&](auto cc_const, int buf) __attribute__((always_inline)) {
            constexpr int cc = decltype(cc_const)::value;
            constexpr int par = cc & 1, hf = cc >> 1;
            uint8_t* dst = stage + buf + me * 2048 + lane * 16;
            asm volatile("" : "+v"(qa[hf]), "+v"(qb[hf]), "+v"(qh[hf]));  // (as for the head)
            const u32x4 xa = par ? qa[hf] >> 4u : qa[hf], xb = par ? qb[hf] >> 4u : qb[hf], xh = par ? qh[hf] >> 4u : qh[hf];
            half2_t s0v[2], c0v[2], s1v[2], c1v[2];  // [low 32 / high 32 of the chunk]
            const uint32_t dw = scl[cc];  // scales 4 cc .. 4 cc + 3: the lane's groups are bytes h and 2 + h
#pragma unroll
            for (int g = 0; g < 2; g++) {
                const int sc = live ? __builtin_amdgcn_sbfe((int)dw, (unsigned)(8 * h + 16 * g), 8u) : 0;
                const float f0 = (float)(sc & 15) * 0.0625f, f1 = (float)(sc >> 4);
                s0v[g] = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_pkrtz(f0, f0));  // (four bits and a power of two: exact)
                s1v[g] = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_pkrtz(f1, f1));
                c0v[g] = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_pkrtz(-1056.0f * f0, -1056.0f * f0));
                c1v[g] = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_pkrtz(-1056.0f * f1, -1056.0f * f1));
            }
#pragma unroll
            for (int s4 = 0; s4 < 4; s4++) {
                const uint32_t x = xa[s4], y = xb[s4], z = xh[s4];
                const uint32_t x8 = x >> 8, y8 = y >> 8, z8 = z >> 8;
                const half2_t t[4] = {
                    __builtin_bit_cast(half2_t, ((z & 0x00030003u) << 4) | ((x & 0x000F000Fu) | 0x64006400u)),
                    __builtin_bit_cast(half2_t, ((z & 0x000C000Cu) << 2) | ((y & 0x000F000Fu) | 0x64006400u)),
                    __builtin_bit_cast(half2_t, ((z8 & 0x00030003u) << 4) | ((x8 & 0x000F000Fu) | 0x64006400u)),
                    __builtin_bit_cast(half2_t, ((z8 & 0x000C000Cu) << 2) | ((y8 & 0x000F000Fu) | 0x64006400u))};
                u32x4 o0, o1;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    o0[e] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(t[e], s0v[e & 1], c0v[e & 1]));
                    o1[e] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(t[e], s1v[e & 1], c1v[e & 1]));
                }
                *reinterpret_cast<u32x4*>(dst + s4 * 8192) = o1;          // part 1: (q - 32) s1
                *reinterpret_cast<u32x4*>(dst + s4 * 8192 + 1024) = o0;   // part 0: (q - 32) s0 / 16
            }
        };
        // While the consumers multiply phase (sb, cc) the producer unpacks the phase two after it -- chunks 2 and 3 of
        // the superblock, then chunks 0 and 1 of the next, whose head it takes up with chunk 0.  Requests, two phases
        // before their use: head and first half of the next superblock with chunk 2, its second half with its chunk 0.
        // (After the last superblock it unpacks a repeat into buffers that nobody reads any more -- no branch, so
        // that the requests are not moved down into one -- and keeps the unit.)
        auto phase = [&](int sb, auto cc_const) __attribute__((always_inline)) {
            constexpr int cc = decltype(cc_const)::value;
            if (cc == 0) {
                load_head(sb + 1);
                load_half(sb + 1, 0);
                unpack(C2{}, b_nx2);
            }
            if (cc == 1) unpack(C3{}, b_nx2);
            if (cc == 2) {
                const float keep = cs;
                enter(sb + 1);
                if (sb + 1 >= nb) cs = keep;
                load_half(sb + 1, 1);
                unpack(C0{}, b_nx2);
            }
            if (cc == 3) unpack(C1{}, b_nx2);
            barrier();
            turn();
        };
        load_head(0);
        load_half(0, 0);
        load_half(0, 1);
        enter(0);
        unpack(C0{}, b_cur);
        unpack(C1{}, b_nxt);
        barrier();
        for (int sb = 0; sb < nb; sb++) {
            phase(sb, C0{});
            phase(sb, C1{});
            phase(sb, C2{});
            phase(sb, C3{});
        }
        if (h == 0) fin[col] = cs;
        barrier();
    } else {
        constexpr int MT = 2;
        const __amdgpu_buffer_rsrc_t arsrc = __builtin_amdgcn_make_buffer_rsrc((void*)afrag, 0, (int)a_bytes, 0x00020000);
        const int mb0 = mt * 8 + me * MT;  // first row block of this consumer
        uint32_t abase[MT];
#pragma unroll
        for (int i = 0; i < MT; i++) abase[i] = (uint32_t)(mb0 + i) * (uint32_t)nch * 4096u;
        u32x4 a[8][MT];  // ring of eight k-steps, seven ahead
        auto afetch = [&](int step, int slot) __attribute__((always_inline)) {  // step: absolute, 16 per superblock
            step = min(step, 16 * nb - 1);  // (past the end: the last step again, unused)
#pragma unroll
            for (int i = 0; i < MT; i++)
                a[slot][i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(arsrc, lane * 16, (int)(abase[i] + (uint32_t)step * 1024u), 0));
        };
        float16_t acc[MT][4];
#pragma unroll
        for (int i = 0; i < MT; i++)
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int x = 0; x < 16; x++) acc[i][j][x] = 0.f;
        // half-step hs = 2 s4 + (part 1 first, then part 0): fragment (s4, j, part) of a phase at (s4 * 8 + j * 2 + p) KiB
        // with p = 0 for part 1; the four fragments of half-step hs + 1 are read while those of hs are multiplied,
        // half-step 0 of a phase in fb[0]
        half8_t fb[2][4];
        float ratio[4] = {1.f, 1.f, 1.f, 1.f};  // of the superblock being entered, by column block
        // tile t = 4 i + j changes its unit: half `part` of its sixteen registers
        auto rescale = [&](int t, int part) __attribute__((always_inline)) {
#pragma unroll
            for (int x = 0; x < 8; x++) acc[t >> 2][t & 3][8 * part + x] *= ratio[t & 3];
        };
        auto fence = [&]() __attribute__((always_inline)) { __builtin_amdgcn_sched_barrier(0); };
        auto phase = [&](int sb, auto cc_const) __attribute__((always_inline)) {
            constexpr int cc = decltype(cc_const)::value;
            const uint8_t* src = stage + b_cur + lane * 16;
            const uint8_t* srcn = stage + b_nxt + lane * 16;
            float rnext[4];
            if (cc == 3) {  // (the ratios of the next superblock, left by the producers a phase ago: used at the end of this phase)
#pragma unroll
                for (int j = 0; j < 4; j++) rnext[j] = ratios[((sb + 1) & 1) * 128 + j * 32 + r];
            }
#pragma unroll
            for (int hs = 0; hs < 8; hs++) {
                const int s4 = hs >> 1, step = 4 * cc + s4, slot = step & 7;
                if (hs < 7) {
                    const int s4n = (hs + 1) >> 1, ptn = (hs + 1) & 1;
#pragma unroll
                    for (int j = 0; j < 4; j++) fb[(hs + 1) & 1][j] = *reinterpret_cast<const half8_t*>(src + s4n * 8192 + j * 2048 + ptn * 1024);
                } else {  // the next phase's first half-step: complete since the barrier before this phase
#pragma unroll
                    for (int j = 0; j < 4; j++) fb[0][j] = *reinterpret_cast<const half8_t*>(srcn + j * 2048);
                }
                if (cc == 3 && hs == 7) {
#pragma unroll
                    for (int j = 0; j < 4; j++) ratio[j] = sb + 1 < nb ? rnext[j] : 1.0f;  // (none after the last superblock)
                }
                fence();
                if ((cc == 0 && hs == 0) || (cc == 3 && hs == 7)) {
                    // the two sides of a superblock's end: tiles 0 .. 2 change their unit between the last matrix
                    // instructions of the superblock, tiles 3 .. 7 between the first of the next
#pragma unroll
                    for (int t = 0; t < 8; t++) {
                        acc[t >> 2][t & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a[slot][t >> 2]), fb[hs & 1][t & 3],
                                                                                    acc[t >> 2][t & 3], 0, 0, 0);
                        fence();
                        if (cc == 3) {
                            if (t >= 2) rescale((t - 2) >> 1, t & 1);
                        } else {
                            if (t < 4) rescale(3 + (t >> 1), t & 1);
                            if (t >= 4 && t < 7) rescale(t + 1, 0), rescale(t + 1, 1);
                        }
                        fence();
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < MT; i++) {
                        const half8_t fa = __builtin_bit_cast(half8_t, a[slot][i]);
#pragma unroll
                        for (int j = 0; j < 4; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa, fb[hs & 1][j], acc[i][j], 0, 0, 0);
                    }
                }
                if (hs & 1) afetch(16 * sb + step + 7, (step + 7) & 7);
                fence();
            }
            barrier();
            turn();
        };
#pragma unroll
        for (int s = 0; s < 7; s++) afetch(s, s);
        barrier();
#pragma unroll
        for (int j = 0; j < 4; j++) fb[0][j] = *reinterpret_cast<const half8_t*>(stage + b_cur + lane * 16 + j * 2048);
        for (int sb = 0; sb < nb; sb++) {
            phase(sb, C0{});
            phase(sb, C1{});
            phase(sb, C2{});
            phase(sb, C3{});
        }
        barrier();
#pragma unroll
        for (int i = 0; i < MT; i++) {
            float sc[16];
#pragma unroll
            for (int x = 0; x < 16; x++) sc[x] = isc_lds[(me * MT + i) * 32 + 8 * (x >> 2) + 4 * h + (x & 3)];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float unit = fin[j * 32 + r];
#pragma unroll
                for (int x = 0; x < 16; x++) acc[i][j][x] *= unit;
                store_tile_scaled(acc[i][j], c, n, (mb0 + i) * 32, n0 + 32 * j, m, n, sc, lane, accumulate != 0);
            }
        }
    }
}

template <int MT>
int launch_q6k_gemm(skn_ctx* ctx, const u32x4* afrag, const uint8_t* w, const float* isc, float* c, int m, int n, int k,
                    int accumulate) {
    constexpr int kLds = 2 * MT * 3 * 4096;
    const int m_tiles = (m + 32 * MT - 1) / (32 * MT), n_tiles = (n + kBN - 1) / kBN;
    const int xcd_rows = 8 % m_tiles == 0 ? 1 : 0;
    const unsigned grid = xcd_rows ? (unsigned)(8 * ((n_tiles + 8 / m_tiles - 1) / (8 / m_tiles))) : (unsigned)(((n_tiles + 7) / 8) * 8 * m_tiles);
    const uint32_t a_bytes = (uint32_t)((size_t)m_tiles * 32 * MT * k * 2);  // (checked by the caller to fit)
    const uint32_t w_bytes = (uint32_t)((size_t)n * (k / 256) * 210);  // (checked by the caller to fit)
    // 128-row tiles: the kernel with specialised wavefronts (measured 6 - 11 % faster); option value 2 keeps to the other
    // (up to 16384 elements per row: a rescale per superblock rounds the accumulators once more, the other form does not)
    if (MT == 4 && xcd_rows && k <= 16384 && ctx->opt_gemm_q6k_fused != 2) {
        skn_launch(ctx, gemm_q6k_pc_kernel, dim3(grid), dim3(512), kQ6PcLds, afrag, w, isc, c, m, n, k, m_tiles, n_tiles, accumulate,
                   a_bytes, w_bytes);
        SKN_LAUNCH_CHECK(ctx);
        return SKN_OK;
    }
    skn_launch(ctx, gemm_q6k_frag_kernel<MT>, dim3(grid), dim3(256), kLds, afrag, w, isc, c, m, n, k, m_tiles, n_tiles, accumulate,
               a_bytes, w_bytes, xcd_rows);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

int launch_q6k_gemm_mt(skn_ctx* ctx, int mt, const u32x4* afrag, const uint8_t* w, const float* isc, float* c, int m, int n,
                       int k, int accumulate) {
    if (mt == 1) return launch_q6k_gemm<1>(ctx, afrag, w, isc, c, m, n, k, accumulate);
    if (mt == 2) return launch_q6k_gemm<2>(ctx, afrag, w, isc, c, m, n, k, accumulate);
    return launch_q6k_gemm<4>(ctx, afrag, w, isc, c, m, n, k, accumulate);
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

// Dynamic LDS above 48 KiB must be allowed per kernel and device; done once per context here so that no launch
// path has to.
int skn_gemm_init(skn_ctx* ctx) {
    SKN_HIP(ctx, hipFuncSetAttribute((const void*)gemm_q4k_frag_kernel<2, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, frag_lds_bytes<2, 2>() + 32 * 2 * 2 * 4));
    SKN_HIP(ctx, hipFuncSetAttribute((const void*)gemm_q4k_frag_kernel<2, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, frag_lds_bytes<2, 1>() + 32 * 2 * 1 * 4));
    SKN_HIP(ctx, hipFuncSetAttribute((const void*)gemm_q4k_tall_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kTlLds));
    SKN_HIP(ctx, hipFuncSetAttribute((const void*)gemm_hilo_frag_kernel<1, 4>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * 1 * 3 * 4096));
    SKN_HIP(ctx, hipFuncSetAttribute((const void*)gemm_hilo_frag_kernel<2, 4>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * 2 * 3 * 4096));
    SKN_HIP(ctx, hipFuncSetAttribute((const void*)gemm_hilo_frag_kernel<4, 4>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * 4 * 3 * 4096));
    SKN_HIP(ctx, hipFuncSetAttribute((const void*)gemm_q6k_tall_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kQ6TlLds));
    SKN_HIP(ctx, hipFuncSetAttribute((const void*)gemm_q6k_pc_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kQ6PcLds));
    SKN_HIP(ctx, hipFuncSetAttribute((const void*)gemm_q6k_frag_kernel<1>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * 1 * 3 * 4096));
    SKN_HIP(ctx, hipFuncSetAttribute((const void*)gemm_q6k_frag_kernel<2>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * 2 * 3 * 4096));
    SKN_HIP(ctx, hipFuncSetAttribute((const void*)gemm_q6k_frag_kernel<4>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * 4 * 3 * 4096));
    return SKN_OK;
}

int skn_gemm_q4k_multi(skn_ctx* ctx, const skn_gemm_seg* segs, int nseg, int k, const skn_gemm_src& src, int m,
                       bool swiglu_pair) {
    SKN_REQUIRE(ctx, nseg >= 1 && nseg <= 3 && m > 0 && k > 0 && k % 256 == 0 && k <= 16384, SKN_ERR_ARG,
                "Q4_K GEMM: bad segment count or shape");
    SKN_REQUIRE(ctx, !swiglu_pair || (nseg == 2 && segs[0].n == segs[1].n && !segs[0].accumulate), SKN_ERR_ARG,
                "Q4_K GEMM: a SwiGLU pair is two matrices of the same shape");
    Q4kFragSegs fs;
    int tiles = 0;
    for (int i = 0; i < 3; i++) {
        const skn_gemm_seg& s = segs[i < nseg ? i : nseg - 1];
        SKN_REQUIRE(ctx, s.w && s.c && s.n > 0 && ((uintptr_t)s.w & 15) == 0, SKN_ERR_ARG,
                    "Q4_K GEMM: weights must be non-null and 16-byte aligned");
        fs.w[i] = (const uint8_t*)s.w, fs.c[i] = s.c, fs.n[i] = s.n, fs.accumulate[i] = s.accumulate, fs.tile0[i] = tiles;
        if (i < nseg) tiles += (s.n + kBN - 1) / kBN;
    }
    for (int i = nseg; i < 3; i++) fs.tile0[i] = tiles;
    fs.n_tiles = swiglu_pair ? (segs[0].n + 31) / 32 : tiles;
    fs.pair = swiglu_pair ? 1 : 0;
    SKN_REQUIRE(ctx, src.a && ((uintptr_t)src.a & (src.kind == SKN_SRC_BF16 ? 7 : 15)) == 0, SKN_ERR_ARG,
                "Q4_K GEMM: activations are null or misaligned");
    SKN_REQUIRE(ctx, src.kind == SKN_SRC_BF16 || src.kind == SKN_SRC_F32 || (src.b && ((uintptr_t)src.b & 15) == 0),
                SKN_ERR_ARG, "Q4_K GEMM: second activation operand is null or misaligned");
    // fragment-order workspace: rows padded to whole tiles
    // Tile rows: 128 (eight wavefronts, one workgroup per compute unit) when that gives at most one tile per
    // compute unit; otherwise 64 with four wavefronts, two independent workgroups per compute unit -- more weight
    // staging per product, but the two wavefronts of a SIMD no longer meet at the same barriers (measured 4-11 %
    // faster on grids of several rounds, 3 % slower on single-round grids).
    const int n_tiles_all = fs.n_tiles;
    // 256 x 128 tiles (the kernel that unpacks the weights once per tile) where they keep at least two thirds of the
    // compute units busy over their rounds: the 14336-column matrices, a q,k,v group and a gate / up pair at 512 rows
    int tall_cols = 0, tall_tile0[3] = {0, 0, 0};
    bool tall_fits = true;
    for (int i = 0; i < nseg; i++) {
        tall_tile0[i] = tall_cols;
        tall_cols += (segs[i].n + 127) / 128;
        tall_fits = tall_fits && (size_t)segs[i].n * (k / 256) * 144 < ((size_t)1 << 31);
    }
    for (int i = nseg; i < 3; i++) tall_tile0[i] = tall_cols;
    if (swiglu_pair) tall_cols = (segs[0].n + 63) / 64;
    const int tall_tiles = ((m + 255) / 256) * tall_cols;
    const int tall_rounds = (tall_tiles + ctx->compute_units - 1) / ctx->compute_units;
    const bool tall = tall_fits && (ctx->opt_gemm_tile == 3 ||
                                    (ctx->opt_gemm_tile == 0 && m > 128 && 3 * tall_tiles >= 2 * tall_rounds * ctx->compute_units));
    const bool small_tiles = !tall && (ctx->opt_gemm_tile == 1 ||
                             (ctx->opt_gemm_tile == 0 && (m <= 128 || ((m + 127) / 128) * n_tiles_all > ctx->compute_units)));
    const int mt_rows = tall ? 256 : small_tiles ? 64 : 128;
    const int m_tiles = (m + mt_rows - 1) / mt_rows, m_pad = m_tiles * mt_rows;
    const size_t af_bytes = align_up((size_t)m_pad * k * 2), sf_bytes = align_up((size_t)m_pad * (k / 256) * 16 * 2);
    SKN_REQUIRE(ctx, af_bytes < ((size_t)1 << 31), SKN_ERR_SHAPE,
                "Q4_K GEMM: %d rows of %d activations exceed the 2^30 elements one call takes", m, k);
    const size_t is_bytes = align_up((size_t)m_pad * 4);
    uint8_t* ws;
    int rc = gemm_workspace(ctx, af_bytes + sf_bytes + is_bytes, &ws);
    if (rc != SKN_OK) return rc;
    _Float16* afrag = (_Float16*)ws;
    _Float16* sfrag = (_Float16*)(ws + af_bytes);
    float* isc = (float*)(ws + af_bytes + sf_bytes);
    switch (src.kind) {
        case SKN_SRC_BF16: launch_prep<SKN_SRC_BF16, true>(ctx, src, afrag, isc, sfrag, m, m_pad, k); break;
        case SKN_SRC_F32: launch_prep<SKN_SRC_F32, true>(ctx, src, afrag, isc, sfrag, m, m_pad, k); break;
        case SKN_SRC_RMSNORM: launch_prep<SKN_SRC_RMSNORM, true>(ctx, src, afrag, isc, sfrag, m, m_pad, k); break;
        default: return skn_fail(ctx, SKN_ERR_ARG, "Q4_K GEMM: unknown activation source %d", src.kind);
    }
    SKN_LAUNCH_CHECK(ctx);
    if (tall) {
        for (int i = 0; i < 3; i++) fs.tile0[i] = tall_tile0[i];
        fs.n_tiles = tall_cols;
        skn_launch(ctx, gemm_q4k_tall_kernel, dim3(m_tiles * tall_cols), dim3(512), kTlLds, (const u32x4*)afrag, (const u32x4*)sfrag, fs, isc, m,
                   k, m_tiles, (uint32_t)((size_t)m_pad * k * 2));
        SKN_LAUNCH_CHECK(ctx);
        return SKN_OK;
    }
    if (mt_rows == 128) return launch_frag<2, 2>(ctx, m_tiles, (const u32x4*)afrag, (const u32x4*)sfrag, fs, isc, m, k);
    return launch_frag<2, 1>(ctx, m_tiles, (const u32x4*)afrag, (const u32x4*)sfrag, fs, isc, m, k);
}

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
    SKN_REQUIRE(ctx, k % 64 == 0, SKN_ERR_SHAPE, "skn_gemm_q: k (%d) must be a multiple of %d", k, 64);

    if (ggml_type == SKN_TYPE_Q4_K && k <= 16384) {
        SKN_REQUIRE(ctx, ((uintptr_t)w_dev & 15) == 0 && ((uintptr_t)a_bf16_dev & 7) == 0, SKN_ERR_ARG,
                    "skn_gemm_q: Q4_K weights must be 16-byte aligned, activations 8-byte aligned");
        const skn_gemm_seg seg = {w_dev, n, c_dev, 0};
        const skn_gemm_src src = {SKN_SRC_BF16, a_bf16_dev, nullptr, 0.f};
        return skn_gemm_q4k_multi(ctx, &seg, 1, k, src, m);
    }

    // general path.  Workspace: activations in fragment order (rows padded to whole tiles) + row scales, then
    // the weights as an fp16 pair in fragment order (rows padded to whole 64-column tiles)
    SKN_REQUIRE(ctx, ((uintptr_t)a_bf16_dev & 7) == 0, SKN_ERR_ARG, "skn_gemm_q: activations must be 8-byte aligned");
    const skn_gemm_src src = {SKN_SRC_BF16, a_bf16_dev, nullptr, 0.f};
    // Q6_K with whole superblocks: the kernels that unpack the blocks themselves (no weight pass, no expanded copy)
    if (ggml_type == SKN_TYPE_Q6_K && skn_gemm_q6k_direct_ok(ctx, n, k, m)) {
        const skn_gemm_seg seg = {w_dev, n, c_dev, 0};
        return skn_gemm_q6k_multi(ctx, &seg, 1, k, src, m);
    }
    const int mt = hilo_mt(m);
    const int m_pad = (m + 32 * mt - 1) / (32 * mt) * (32 * mt), n_pad = (n + kBN - 1) / kBN * kBN;
    const size_t af_bytes = align_up((size_t)m_pad * k * 2), is_bytes = align_up((size_t)m_pad * 4);
    uint8_t* ws;
    int rc = gemm_workspace(ctx, af_bytes + is_bytes + (size_t)n_pad * k * 4, &ws);
    if (rc != SKN_OK) return rc;
    _Float16* afrag = (_Float16*)ws;
    float* isc = (float*)(ws + af_bytes);
    uint8_t* bfrag = ws + af_bytes + is_bytes;
    _Float16* no_sums = nullptr;
    launch_prep<SKN_SRC_BF16, false>(ctx, src, afrag, isc, no_sums, m, m_pad, k);
    SKN_LAUNCH_CHECK(ctx);
    rc = skn_weights_hilo_frag(ctx, ggml_type, (const uint8_t*)w_dev, n, k, bfrag);
    if (rc != SKN_OK) return rc;
    return launch_hilo_gemm_mt(ctx, mt, (const u32x4*)afrag, (const u32x4*)bfrag, isc, c_dev, m, n, k, 0);
}

namespace {
// 256 x 128 tiles for a Q6_K matrix: where they fill three quarters of the compute units or more in one round (or by option)
bool q6k_wide_tiles(const skn_ctx* ctx, int n, int k, int m) {
    const int tiles = ((m + 255) / 256) * ((n + 127) / 128);
    return k <= 16384 && ctx->opt_gemm_q6k_fused == 1 &&
           (ctx->opt_gemm_tile == 3 ||
            (ctx->opt_gemm_tile == 0 && m > 128 && 4 * tiles >= 3 * ctx->compute_units && tiles <= ctx->compute_units));
}
}  // namespace

bool skn_gemm_q6k_direct_ok(const skn_ctx* ctx, int n, int k, int m) {
    const size_t m_pad = ((size_t)m + 255) / 256 * 256;
    return ctx->opt_gemm_q6k_fused != 0 && n > 0 && m > 0 && k > 0 && k % 256 == 0 && m_pad * k * 2 + 256 < ((size_t)1 << 31) &&
           (size_t)n * (k / 256) * 210 < ((size_t)1 << 31);
}

int skn_gemm_q6k_multi(skn_ctx* ctx, const skn_gemm_seg* segs, int nseg, int k, const skn_gemm_src& src, int m) {
    SKN_REQUIRE(ctx, nseg >= 1 && nseg <= 3 && m > 0, SKN_ERR_ARG, "Q6_K GEMM: bad segment count or shape");
    SKN_REQUIRE(ctx, src.a && ((uintptr_t)src.a & (src.kind == SKN_SRC_BF16 ? 7 : 15)) == 0, SKN_ERR_ARG,
                "Q6_K GEMM: activations are null or misaligned");
    SKN_REQUIRE(ctx, src.kind == SKN_SRC_BF16 || src.kind == SKN_SRC_F32 || (src.b && ((uintptr_t)src.b & 15) == 0),
                SKN_ERR_ARG, "Q6_K GEMM: second activation operand is null or misaligned");
    bool any_wide = false;
    for (int i = 0; i < nseg; i++) {
        SKN_REQUIRE(ctx, segs[i].w && segs[i].c && skn_gemm_q6k_direct_ok(ctx, segs[i].n, k, m), SKN_ERR_ARG,
                    "Q6_K GEMM: a matrix is null or not one this path takes");
        any_wide = any_wide || q6k_wide_tiles(ctx, segs[i].n, k, m);
    }
    // (rows padded to the tallest tile in use: the kernels with shorter tiles address their own row blocks inside it)
    const int mt = hilo_mt(m);
    const int m_rows = any_wide ? 256 : 32 * mt;
    const int m_pad = (m + m_rows - 1) / m_rows * m_rows;
    const size_t af_bytes = align_up((size_t)m_pad * k * 2), is_bytes = align_up((size_t)m_pad * 4);
    uint8_t* ws;
    int rc = gemm_workspace(ctx, af_bytes + is_bytes, &ws);
    if (rc != SKN_OK) return rc;
    _Float16* afrag = (_Float16*)ws;
    float* isc = (float*)(ws + af_bytes);
    _Float16* no_sums = nullptr;
    switch (src.kind) {
        case SKN_SRC_BF16: launch_prep<SKN_SRC_BF16, false>(ctx, src, afrag, isc, no_sums, m, m_pad, k); break;
        case SKN_SRC_F32: launch_prep<SKN_SRC_F32, false>(ctx, src, afrag, isc, no_sums, m, m_pad, k); break;
        case SKN_SRC_RMSNORM: launch_prep<SKN_SRC_RMSNORM, false>(ctx, src, afrag, isc, no_sums, m, m_pad, k); break;
        default: return skn_fail(ctx, SKN_ERR_ARG, "Q6_K GEMM: unknown activation source %d", src.kind);
    }
    SKN_LAUNCH_CHECK(ctx);
    for (int i = 0; i < nseg; i++) {
        const int n = segs[i].n;
        if (q6k_wide_tiles(ctx, n, k, m)) {
            const int m_tiles = m_pad / 256, tiles = m_tiles * ((n + 127) / 128);
            skn_launch(ctx, gemm_q6k_tall_kernel, dim3((unsigned)tiles), dim3(512), kQ6TlLds, (const u32x4*)afrag, (const uint8_t*)segs[i].w,
                       (const float*)isc, segs[i].c, m, n, k, m_tiles, segs[i].accumulate, (uint32_t)((size_t)m_pad * k * 2),
                       (uint32_t)((size_t)n * (k / 256) * 210));
            SKN_LAUNCH_CHECK(ctx);
        } else {
            rc = launch_q6k_gemm_mt(ctx, mt, (const u32x4*)afrag, (const uint8_t*)segs[i].w, isc, segs[i].c, m, n, k, segs[i].accumulate);
            if (rc != SKN_OK) return rc;
        }
    }
    return SKN_OK;
}

// ---- expanded weights: the general path with its weight pass done once ------------------------------------
// The fp16-pair copy of a weight matrix that the general path builds per call (4 bytes per weight, rows padded to
// whole 64-column tiles) can be kept by the caller: skn_gemm_expand fills it, skn_gemm_expanded multiplies with it.

size_t skn_gemm_expanded_size(int n, int k) { return (size_t)((n + kBN - 1) / kBN * kBN) * (size_t)k * 4; }

int skn_gemm_expanded_multi(skn_ctx* ctx, const skn_gemm_seg* segs, int nseg, int k, const skn_gemm_src& src, int m) {
    SKN_REQUIRE(ctx, nseg >= 1 && m > 0 && k > 0 && k % 64 == 0, SKN_ERR_ARG, "expanded GEMM: bad segment count or shape");
    SKN_REQUIRE(ctx, src.a && ((uintptr_t)src.a & (src.kind == SKN_SRC_BF16 ? 7 : 15)) == 0, SKN_ERR_ARG,
                "expanded GEMM: activations are null or misaligned");
    SKN_REQUIRE(ctx, src.kind == SKN_SRC_BF16 || src.kind == SKN_SRC_F32 || (src.b && ((uintptr_t)src.b & 15) == 0),
                SKN_ERR_ARG, "expanded GEMM: second activation operand is null or misaligned");
    for (int i = 0; i < nseg; i++)
        SKN_REQUIRE(ctx, segs[i].w && segs[i].c && segs[i].n > 0 && ((uintptr_t)segs[i].w & 15) == 0, SKN_ERR_ARG,
                    "expanded GEMM: weights must be non-null and 16-byte aligned");
    const int mt = hilo_mt(m);
    const int m_pad = (m + 32 * mt - 1) / (32 * mt) * (32 * mt);
    const size_t af_bytes = align_up((size_t)m_pad * k * 2), is_bytes = align_up((size_t)m_pad * 4);
    SKN_REQUIRE(ctx, af_bytes < ((size_t)1 << 31), SKN_ERR_SHAPE,
                "expanded GEMM: %d rows of %d activations exceed the 2^30 elements one call takes", m, k);
    uint8_t* ws;
    int rc = gemm_workspace(ctx, af_bytes + is_bytes, &ws);
    if (rc != SKN_OK) return rc;
    _Float16* afrag = (_Float16*)ws;
    float* isc = (float*)(ws + af_bytes);
    _Float16* no_sums = nullptr;
    switch (src.kind) {
        case SKN_SRC_BF16: launch_prep<SKN_SRC_BF16, false>(ctx, src, afrag, isc, no_sums, m, m_pad, k); break;
        case SKN_SRC_F32: launch_prep<SKN_SRC_F32, false>(ctx, src, afrag, isc, no_sums, m, m_pad, k); break;
        case SKN_SRC_RMSNORM: launch_prep<SKN_SRC_RMSNORM, false>(ctx, src, afrag, isc, no_sums, m, m_pad, k); break;
        default: return skn_fail(ctx, SKN_ERR_ARG, "expanded GEMM: unknown activation source %d", src.kind);
    }
    SKN_LAUNCH_CHECK(ctx);
    for (int i = 0; i < nseg; i++) {
        rc = launch_hilo_gemm_mt(ctx, mt, (const u32x4*)afrag, (const u32x4*)segs[i].w, isc, segs[i].c, m, segs[i].n, k,
                                 segs[i].accumulate);
        if (rc != SKN_OK) return rc;
    }
    return SKN_OK;
}

extern "C" int skn_gemm_expanded_bytes(skn_ctx* ctx, int ggml_type, int n, int k, size_t* bytes_out) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_gemm_expanded_bytes: ctx is null");
    SKN_REQUIRE(ctx, bytes_out != nullptr, SKN_ERR_ARG, "skn_gemm_expanded_bytes: bytes_out is null");
    SKN_REQUIRE(ctx, skn_is_quant(ggml_type), SKN_ERR_TYPE, "skn_gemm_expanded_bytes: ggml type %d is not supported", ggml_type);
    SKN_REQUIRE(ctx, n >= 0 && k >= 0, SKN_ERR_ARG, "skn_gemm_expanded_bytes: negative shape");
    int be, bb;
    skn_type_block(ggml_type, &be, &bb);
    SKN_REQUIRE(ctx, k % be == 0, SKN_ERR_SHAPE, "Quantized tensor row size (%d) is not a multiple of block size (%d)", k,
                be);
    SKN_REQUIRE(ctx, k % 64 == 0, SKN_ERR_SHAPE, "skn_gemm_expanded_bytes: k (%d) must be a multiple of %d", k, 64);
    *bytes_out = skn_gemm_expanded_size(n, k);
    return SKN_OK;
}

extern "C" int skn_gemm_expand(skn_ctx* ctx, int ggml_type, const void* w_dev, int n, int k, void* expanded_dev) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_gemm_expand: ctx is null");
    size_t bytes = 0;
    int rc = skn_gemm_expanded_bytes(ctx, ggml_type, n, k, &bytes);
    if (rc != SKN_OK) return rc;
    if (bytes == 0) return SKN_OK;
    SKN_REQUIRE(ctx, w_dev && expanded_dev, SKN_ERR_ARG, "skn_gemm_expand: null pointer");
    SKN_REQUIRE(ctx, ((uintptr_t)expanded_dev & 15) == 0, SKN_ERR_ARG, "skn_gemm_expand: the copy must be 16-byte aligned");
    return skn_weights_hilo_frag(ctx, ggml_type, (const uint8_t*)w_dev, n, k, expanded_dev);
}

extern "C" int skn_gemm_expanded(skn_ctx* ctx, const void* expanded_dev, int n, int k, const uint16_t* a_bf16_dev, int m,
                                 float* c_dev) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_gemm_expanded: ctx is null");
    SKN_REQUIRE(ctx, n >= 0 && k >= 0 && m >= 0, SKN_ERR_ARG, "skn_gemm_expanded: negative shape");
    SKN_REQUIRE(ctx, k % 64 == 0, SKN_ERR_SHAPE, "skn_gemm_expanded: k (%d) must be a multiple of %d", k, 64);
    if (n == 0 || m == 0) return SKN_OK;
    SKN_REQUIRE(ctx, c_dev != nullptr, SKN_ERR_ARG, "skn_gemm_expanded: c is null");
    if (k == 0) return skn_memset(ctx, c_dev, 0, (size_t)m * n * sizeof(float));
    SKN_REQUIRE(ctx, expanded_dev && a_bf16_dev, SKN_ERR_ARG, "skn_gemm_expanded: null pointer");
    const skn_gemm_seg seg = {expanded_dev, n, c_dev, 0};
    const skn_gemm_src src = {SKN_SRC_BF16, a_bf16_dev, nullptr, 0.f};
    return skn_gemm_expanded_multi(ctx, &seg, 1, k, src, m);
}
