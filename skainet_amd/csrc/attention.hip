// Decode attention over the paged KV cache: out[s,h,:] = softmax(q[s,h,:] . K^T * scale) . V.
//
// One query row per (sequence, head), so every K and V byte is used exactly once: the kernel is an HBM
// stream of 2 * n_ctx * head_dim * 2 bytes per (sequence, head) at 1 flop per byte.  The context is split
// across workgroups (flash-decoding): grid = (splits, heads, sequences).
//
// Inside a workgroup there is no staging and no barrier while tokens stream: a token row (head_dim halves)
// is spread over head_dim / 8 consecutive lanes, 16 bytes each, so one wavefront load instruction covers
// 64 * 8 / head_dim consecutive tokens (1 KiB contiguous in a page).  The lanes of a token form a group that
// owns a private softmax stream: the score is the group's DPP all-reduce of eight products per lane, every
// lane of the group then holds the same (running max, running sum) and its own eight output dimensions, and
// the V row is loaded with the same lane mapping as the K row.  The streams of a workgroup are merged once at
// the end through LDS; the partials of the splits are merged by whichever workgroup of a (sequence, head)
// finishes last (a counter in device memory, reset by that workgroup), so the whole step is one launch.
#include "kv.h"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

constexpr int kAttnThreads = 256;
constexpr int kMaxSplits = 512;
constexpr int kUnroll = 4;  // tokens per stream in flight per iteration (K and V: 8 x 16 bytes per lane)

template <int LPT>
__device__ __forceinline__ float group_sum(float v) {
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xF, 0xF, true));   // lane ^ 1
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xF, 0xF, true));   // lane ^ 2
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x141, 0xF, 0xF, true));  // 7 - lane
    if constexpr (LPT >= 16) v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x140, 0xF, 0xF, true));
    if constexpr (LPT >= 32) v += __shfl_xor(v, 16, 64);
    return v;
}

__device__ __forceinline__ float dot8(const u32x4& k, const float (&qf)[8]) {
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint32_t w = k[j];  // (a bit cast applied directly to a vector element reads element 0)
        const half2_t h = __builtin_bit_cast(half2_t, w);
        s = fmaf((float)h.x, qf[2 * j], s);
        s = fmaf((float)h.y, qf[2 * j + 1], s);
    }
    return s;
}

template <int D, bool POW2>
__global__ __launch_bounds__(kAttnThreads) void attn_decode_kernel(
    const uint16_t* __restrict__ k_pool, const uint16_t* __restrict__ v_pool, const int32_t* __restrict__ table,
    const int32_t* __restrict__ nctx, const float* __restrict__ q, float* partial, int* counters, float* __restrict__ out,
    int n_head, int kv_heads, int page_tokens, int page_shift, int pages_per_seq, int n_splits, float scale, int seq_fixed) {
    constexpr int LPT = D / 8;                        // lanes per token
    constexpr int G = 64 / LPT;                       // token groups (streams) per wavefront
    constexpr int NS = (kAttnThreads / 64) * G;       // streams per workgroup
    constexpr int U = kUnroll;
    __shared__ float so[NS][D];
    __shared__ float sm[NS], sl[NS];
    __shared__ float pm[kMaxSplits], pl[kMaxSplits];
    __shared__ int last_flag;
    static_assert(kAttnThreads / (D / 4) <= NS, "the split merge reuses the stream rows");

    // blockIdx.z is the query row: its own sequence by default, or one shared sequence (seq_fixed >= 0) when
    // several query rows attend to prefixes of the same cache (prompt processing)
    const int split = blockIdx.x, h = blockIdx.y, s = blockIdx.z;
    // grouped queries: n_head query heads share kv_heads cached heads, n_head / kv_heads consecutive ones each
    const int kvh = kv_heads == n_head ? h : h / (n_head / kv_heads);
    const int kv_seq = seq_fixed >= 0 ? seq_fixed : s;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = lane % LPT, g = lane / LPT;
    const int stream = wave * G + g;
    const int n = nctx[s];
    const int per = ((n + n_splits - 1) / n_splits + NS - 1) / NS * NS;  // whole wavefront loads per split
    const int t_begin = split * per;
    const int t_end = min(n, t_begin + per);

    float qf[8];
    {
        const float4* qp = reinterpret_cast<const float4*>(q + ((size_t)s * n_head + h) * D + c * 8);
        const float4 a = qp[0], b = qp[1];
        qf[0] = a.x * scale, qf[1] = a.y * scale, qf[2] = a.z * scale, qf[3] = a.w * scale;
        qf[4] = b.x * scale, qf[5] = b.y * scale, qf[6] = b.z * scale, qf[7] = b.w * scale;
    }
    float o[8];
#pragma unroll
    for (int j = 0; j < 8; j++) o[j] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;
    const int32_t* trow = table + (size_t)kv_seq * pages_per_seq;
    // the first 64 page ids of the sequence ride in a register (lane i holds page i), fetched here together with
    // the length and the query instead of once the token range is known: one dependent round trip less
    const int my_page = trow[min(lane, pages_per_seq - 1)];

    for (int base = t_begin; base < t_end; base += NS * U) {
        u32x4 kk[U], vv[U];
        bool ok[U];
        int page[U], slot[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int t = base + u * NS + stream;
            ok[u] = t < t_end;
            const int tc = min(t, t_end - 1);  // past the end: a valid row, masked below
            const int pi = POW2 ? tc >> page_shift : tc / page_tokens;
            slot[u] = tc - pi * page_tokens;
            page[u] = __shfl(my_page, pi & 63, 64);
            if (pi >= 64) page[u] = trow[pi];
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const size_t off = (((size_t)page[u] * kv_heads + kvh) * page_tokens + slot[u]) * D + c * 8;
            kk[u] = *reinterpret_cast<const u32x4*>(k_pool + off);
            vv[u] = *reinterpret_cast<const u32x4*>(v_pool + off);
        }
        float sc[U];
        float m_new = m_run;
#pragma unroll
        for (int u = 0; u < U; u++) {
            const float d = group_sum<LPT>(dot8(kk[u], qf));
            sc[u] = ok[u] ? d : -INFINITY;
            m_new = fmaxf(m_new, sc[u]);
        }
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;  // keeps exp(-inf - -inf) out of the arithmetic
        const float alpha = __expf(m_run - m_safe);
        float p[U], psum = 0.f;
#pragma unroll
        for (int u = 0; u < U; u++) {
            p[u] = __expf(sc[u] - m_safe);
            psum += p[u];
        }
        l_run = fmaf(l_run, alpha, psum);
        m_run = m_new;
#pragma unroll
        for (int j = 0; j < 8; j++) o[j] *= alpha;
#pragma unroll
        for (int u = 0; u < U; u++) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t w = vv[u][j];
                const half2_t hv = __builtin_bit_cast(half2_t, w);
                o[2 * j] = fmaf(p[u], (float)hv.x, o[2 * j]);
                o[2 * j + 1] = fmaf(p[u], (float)hv.y, o[2 * j + 1]);
            }
        }
    }

    // merge the streams of the workgroup
#pragma unroll
    for (int j = 0; j < 8; j++) so[stream][c * 8 + j] = o[j];
    if (c == 0) {
        sm[stream] = m_run;
        sl[stream] = l_run;
    }
    __syncthreads();
    const int pair = s * n_head + h;
    float M = -INFINITY, acc = 0.f, L = 0.f;
    if (tid < D) {
#pragma unroll
        for (int i = 0; i < NS; i++) M = fmaxf(M, sm[i]);
        const float m_safe = M == -INFINITY ? 0.f : M;
#pragma unroll
        for (int i = 0; i < NS; i++) {
            const float wgt = __expf(sm[i] - m_safe);
            acc = fmaf(wgt, so[i][tid], acc);
            L = fmaf(wgt, sl[i], L);
        }
    }
    if (n_splits == 1) {
        if (tid < D) out[(size_t)pair * D + tid] = L > 0.f ? acc / L : 0.f;
        return;
    }
    // partial: per (pair, split) D + 2 floats: unnormalised output, max, sum
    float* mine = partial + ((size_t)pair * n_splits + split) * (D + 2);
    // Partials and counters are written and read as device-scope atomics (relaxed): such stores go through to
    // the level all compute dies share and such loads never hit a stale line, so no cache-wide write-back or
    // invalidate is needed; order comes from waiting for the stores (vmcnt) before the barrier that precedes
    // the counter increment.
    if (tid < D) __hip_atomic_store(&mine[tid], acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (tid == 0) {
        __hip_atomic_store(&mine[D], M, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&mine[D + 1], L, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    // the last workgroup of this (sequence, head) to get here merges the splits
    if (tid == 0)
        last_flag = __hip_atomic_fetch_add(&counters[pair], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == n_splits - 1;
    __syncthreads();
    if (!last_flag) return;
    // split maxima and sums into LDS with one round of loads, then rows of partial outputs as float4:
    // D / 4 threads per split row, P rows in flight
    const float* base_p = partial + (size_t)pair * n_splits * (D + 2);
    for (int i = tid; i < n_splits; i += kAttnThreads) {
        pm[i] = __hip_atomic_load(&base_p[i * (D + 2) + D], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        pl[i] = __hip_atomic_load(&base_p[i * (D + 2) + D + 1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();  // also: every thread is past the stream merge, so / sl are free again
    float M2 = -INFINITY;
    for (int i = 0; i < n_splits; i++) M2 = fmaxf(M2, pm[i]);
    const float m2_safe = M2 == -INFINITY ? 0.f : M2;
    constexpr int DV = D / 4, P = kAttnThreads / DV;
    const int dq = tid % DV, part = tid / DV;
    float4 a4 = make_float4(0.f, 0.f, 0.f, 0.f);
    float L2 = 0.f;
#pragma unroll 4
    for (int i = part; i < n_splits; i += P) {
        const float wgt = __expf(pm[i] - m2_safe);
        // rows are 8-byte aligned: two 64-bit loads per thread
        const unsigned long long* row = reinterpret_cast<const unsigned long long*>(base_p + (size_t)i * (D + 2)) + 2 * dq;
        const unsigned long long u0 = __hip_atomic_load(row, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned long long u1 = __hip_atomic_load(row + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const float2 lo = make_float2(__uint_as_float((uint32_t)u0), __uint_as_float((uint32_t)(u0 >> 32)));
        const float2 hi = make_float2(__uint_as_float((uint32_t)u1), __uint_as_float((uint32_t)(u1 >> 32)));
        a4.x = fmaf(wgt, lo.x, a4.x);
        a4.y = fmaf(wgt, lo.y, a4.y);
        a4.z = fmaf(wgt, hi.x, a4.z);
        a4.w = fmaf(wgt, hi.y, a4.w);
        L2 = fmaf(wgt, pl[i], L2);
    }
    *reinterpret_cast<float4*>(&so[part][dq * 4]) = a4;
    if (dq == 0) sl[part] = L2;
    __syncthreads();
    if (tid < D) {
        float acc2 = 0.f;
        L2 = 0.f;
#pragma unroll
        for (int i = 0; i < P; i++) {
            acc2 += so[i][tid];
            L2 += sl[i];
        }
        out[(size_t)pair * D + tid] = L2 > 0.f ? acc2 / L2 : 0.f;
    }
    if (tid == 0) __hip_atomic_store(&counters[pair], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
}


// The same streams on sixteen wavefronts, for the decoder's step: a workgroup's token range (up to 256 tokens at
// head_dim 128) is requested in one go, the streams of a wavefront merge through lane exchanges and the sixteen
// wavefronts through LDS -- and that is all: with more than one split the workgroup leaves its unnormalised output and
// its (max, sum) in memory with ordinary stores and ends.  Whoever reads them next merges them (the output
// projection's staging, csrc/matvec.hip), so the launch has no device-wide counter, no waiting for stores and no
// second round of loads behind one.
constexpr int kWideThreads = 1024;

template <int D, bool POW2>
__global__ __launch_bounds__(kWideThreads) void attn_decode_wide_kernel(
    const uint16_t* __restrict__ k_pool, const uint16_t* __restrict__ v_pool, const int32_t* __restrict__ table,
    const int32_t* __restrict__ nctx, const float* __restrict__ q, float* __restrict__ opart, float* __restrict__ ml,
    float* __restrict__ out, int n_head, int kv_heads, int page_tokens, int page_shift, int pages_per_seq, int n_splits,
    float scale, int seq_fixed) {
    constexpr int LPT = D / 8, G = 64 / LPT, W = kWideThreads / 64, NS = W * G, U = kUnroll;
    __shared__ float so[W][D];
    __shared__ float sm[W], sl[W];
    const int split = blockIdx.x, h = blockIdx.y, s = blockIdx.z;
    const int kvh = kv_heads == n_head ? h : h / (n_head / kv_heads);
    const int kv_seq = seq_fixed >= 0 ? seq_fixed : s;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = lane % LPT, g = lane / LPT;
    const int stream = wave * G + g;
    const int n = nctx[s];
    const int per = ((n + n_splits - 1) / n_splits + NS - 1) / NS * NS;
    const int t_begin = split * per;
    const int t_end = min(n, t_begin + per);

    float qf[8];
    {
        const float4* qp = reinterpret_cast<const float4*>(q + ((size_t)s * n_head + h) * D + c * 8);
        const float4 a = qp[0], b = qp[1];
        qf[0] = a.x * scale, qf[1] = a.y * scale, qf[2] = a.z * scale, qf[3] = a.w * scale;
        qf[4] = b.x * scale, qf[5] = b.y * scale, qf[6] = b.z * scale, qf[7] = b.w * scale;
    }
    float o[8];
#pragma unroll
    for (int j = 0; j < 8; j++) o[j] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;
    const int32_t* trow = table + (size_t)kv_seq * pages_per_seq;
    const int my_page = trow[min(lane, pages_per_seq - 1)];

    for (int base = t_begin; base < t_end; base += NS * U) {
        u32x4 kk[U], vv[U];
        bool ok[U];
        int page[U], slot[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int t = base + u * NS + stream;
            ok[u] = t < t_end;
            const int tc = min(t, t_end - 1);
            const int pi = POW2 ? tc >> page_shift : tc / page_tokens;
            slot[u] = tc - pi * page_tokens;
            page[u] = __shfl(my_page, pi & 63, 64);
            if (pi >= 64) page[u] = trow[pi];
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const size_t off = (((size_t)page[u] * kv_heads + kvh) * page_tokens + slot[u]) * D + c * 8;
            kk[u] = *reinterpret_cast<const u32x4*>(k_pool + off);
            vv[u] = *reinterpret_cast<const u32x4*>(v_pool + off);
        }
        float sc[U];
        float m_new = m_run;
#pragma unroll
        for (int u = 0; u < U; u++) {
            const float d = group_sum<LPT>(dot8(kk[u], qf));
            sc[u] = ok[u] ? d : -INFINITY;
            m_new = fmaxf(m_new, sc[u]);
        }
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __expf(m_run - m_safe);
        float p[U], psum = 0.f;
#pragma unroll
        for (int u = 0; u < U; u++) {
            p[u] = __expf(sc[u] - m_safe);
            psum += p[u];
        }
        l_run = fmaf(l_run, alpha, psum);
        m_run = m_new;
#pragma unroll
        for (int j = 0; j < 8; j++) o[j] *= alpha;
#pragma unroll
        for (int u = 0; u < U; u++) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t w = vv[u][j];
                const half2_t hv = __builtin_bit_cast(half2_t, w);
                o[2 * j] = fmaf(p[u], (float)hv.x, o[2 * j]);
                o[2 * j + 1] = fmaf(p[u], (float)hv.y, o[2 * j + 1]);
            }
        }
    }
    // the G streams of the wavefront: lanes with the same c hold the same dimensions
    float mw = m_run;
#pragma unroll
    for (int off = LPT; off < 64; off <<= 1) mw = fmaxf(mw, __shfl_xor(mw, off, 64));
    const float mw_safe = mw == -INFINITY ? 0.f : mw;
    const float wg = __expf(m_run - mw_safe);  // (an empty stream: exp(-inf) = 0)
    float lw = l_run * wg;
#pragma unroll
    for (int j = 0; j < 8; j++) o[j] *= wg;
#pragma unroll
    for (int off = LPT; off < 64; off <<= 1) {
        lw += __shfl_xor(lw, off, 64);
#pragma unroll
        for (int j = 0; j < 8; j++) o[j] += __shfl_xor(o[j], off, 64);
    }
    if (g == 0) {
#pragma unroll
        for (int j = 0; j < 8; j++) so[wave][c * 8 + j] = o[j];
        if (c == 0) {
            sm[wave] = mw;
            sl[wave] = lw;
        }
    }
    __syncthreads();
    if (tid < D) {
        float M = -INFINITY, acc = 0.f, L = 0.f;
#pragma unroll
        for (int i = 0; i < W; i++) M = fmaxf(M, sm[i]);
        const float m_safe = M == -INFINITY ? 0.f : M;
#pragma unroll
        for (int i = 0; i < W; i++) {
            const float wgt = __expf(sm[i] - m_safe);
            acc = fmaf(wgt, so[i][tid], acc);
            L = fmaf(wgt, sl[i], L);
        }
        const int pair = s * n_head + h, n_pairs = gridDim.z * n_head;
        if (n_splits == 1) {
            out[(size_t)pair * D + tid] = L > 0.f ? acc / L : 0.f;
        } else {
            opart[((size_t)split * n_pairs + pair) * D + tid] = acc;
            if (tid == 0) {
                ml[2 * ((size_t)split * n_pairs + pair)] = M;
                ml[2 * ((size_t)split * n_pairs + pair) + 1] = L;
            }
        }
    }
}

}  // namespace

// Shared with the decoder.  n_queries query rows; row z attends to nctx_dev[z] tokens of sequence z
// (seq_fixed < 0) or of sequence seq_fixed.  With more than one split, `partial` holds n_queries * n_head *
// n_splits * (head_dim + 2) floats and `counters` n_queries * n_head ints that are zero between launches:
// zeroed once by their owner, left zero by every launch.
int skn_attn_launch_ex(skn_ctx* ctx, skn_kv* kv, const float* q_dev, const int32_t* nctx_dev, int n_queries,
                       int seq_fixed, int n_splits, float* partial, int* counters, float scale, float* out_dev,
                       int n_q_head) {
    const int D = kv->head_dim;
    if (n_q_head <= 0) n_q_head = kv->n_head;
    SKN_REQUIRE(ctx, n_q_head % kv->n_head == 0, SKN_ERR_SHAPE,
                "attention: %d query heads are not a multiple of the %d cached heads", n_q_head, kv->n_head);
    SKN_REQUIRE(ctx, D == 64 || D == 128 || D == 256, SKN_ERR_SHAPE,
                "skn_attn_decode: head_dim %d is not supported (64, 128 or 256)", D);
    SKN_REQUIRE(ctx, n_splits <= kMaxSplits, SKN_ERR_ARG, "skn_attn_decode: %d splits (at most %d)", n_splits, kMaxSplits);
    SKN_REQUIRE(ctx, n_splits >= 1 && (n_splits == 1 || (partial != nullptr && counters != nullptr)), SKN_ERR_ARG,
                "skn_attn_decode: %d splits without scratch", n_splits);
    int page_shift = -1;
    if ((kv->page_tokens & (kv->page_tokens - 1)) == 0)
        for (page_shift = 0; (1 << page_shift) < kv->page_tokens; page_shift++) {}
    dim3 grid(n_splits, n_q_head, n_queries), block(kAttnThreads);
#define SKN_ATTN_LAUNCH(DD)                                                                                        \
    do {                                                                                                           \
        if (page_shift >= 0)                                                                                       \
            skn_launch(ctx, attn_decode_kernel<DD, true>, grid, block, 0, kv->k_pool, kv->v_pool,                  \
                       kv->page_table_dev, nctx_dev, q_dev, partial, counters, out_dev, n_q_head, kv->n_head,      \
                       kv->page_tokens, page_shift, kv->pages_per_seq, n_splits, scale, seq_fixed);                \
        else                                                                                                       \
            skn_launch(ctx, attn_decode_kernel<DD, false>, grid, block, 0, kv->k_pool, kv->v_pool,                 \
                       kv->page_table_dev, nctx_dev, q_dev, partial, counters, out_dev, n_q_head, kv->n_head,      \
                       kv->page_tokens, page_shift, kv->pages_per_seq, n_splits, scale, seq_fixed);                \
    } while (0)
    if (D == 64) SKN_ATTN_LAUNCH(64);
    else if (D == 128) SKN_ATTN_LAUNCH(128);
    else SKN_ATTN_LAUNCH(256);
#undef SKN_ATTN_LAUNCH
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

int skn_attn_launch_unmerged(skn_ctx* ctx, skn_kv* kv, const float* q_dev, const int32_t* nctx_dev, int n_queries,
                             int seq_fixed, int n_splits, float* opart, float* ml, float scale, float* out_dev, int n_q_head) {
    const int D = kv->head_dim;
    if (n_q_head <= 0) n_q_head = kv->n_head;
    SKN_REQUIRE(ctx, n_q_head % kv->n_head == 0, SKN_ERR_SHAPE,
                "attention: %d query heads are not a multiple of the %d cached heads", n_q_head, kv->n_head);
    SKN_REQUIRE(ctx, D == 64 || D == 128 || D == 256, SKN_ERR_SHAPE, "attention: head_dim %d is not supported (64, 128 or 256)", D);
    SKN_REQUIRE(ctx, n_splits >= 1 && (n_splits == 1 ? out_dev != nullptr : (opart != nullptr && ml != nullptr)), SKN_ERR_ARG,
                "attention: %d splits without their buffers", n_splits);
    int page_shift = -1;
    if ((kv->page_tokens & (kv->page_tokens - 1)) == 0)
        for (page_shift = 0; (1 << page_shift) < kv->page_tokens; page_shift++) {}
    dim3 grid(n_splits, n_q_head, n_queries), block(kWideThreads);
#define SKN_ATTN_WIDE(DD)                                                                                              \
    do {                                                                                                               \
        if (page_shift >= 0)                                                                                           \
            skn_launch(ctx, attn_decode_wide_kernel<DD, true>, grid, block, 0, kv->k_pool, kv->v_pool, kv->page_table_dev, \
                       nctx_dev, q_dev, opart, ml, out_dev, n_q_head, kv->n_head, kv->page_tokens, page_shift,         \
                       kv->pages_per_seq, n_splits, scale, seq_fixed);                                                 \
        else                                                                                                           \
            skn_launch(ctx, attn_decode_wide_kernel<DD, false>, grid, block, 0, kv->k_pool, kv->v_pool, kv->page_table_dev, \
                       nctx_dev, q_dev, opart, ml, out_dev, n_q_head, kv->n_head, kv->page_tokens, page_shift,         \
                       kv->pages_per_seq, n_splits, scale, seq_fixed);                                                 \
    } while (0)
    if (D == 64) SKN_ATTN_WIDE(64);
    else if (D == 128) SKN_ATTN_WIDE(128);
    else SKN_ATTN_WIDE(256);
#undef SKN_ATTN_WIDE
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

int skn_attn_splits(skn_ctx* ctx, int pairs, int max_ctx) {
    const int chunks = (max_ctx + 63) / 64;  // a split should hold at least one full iteration of a workgroup
    // One workgroup per compute unit in all: measured over (sequences x heads, context) from 16 x 8192 to 512 x 4096,
    // the fastest split count was compute_units / pairs every time -- 8 x 32 x 4096 takes 88 us with one split and
    // 98 - 103 us with four, 1 x 32 x 4096 14.0 us with eight and 19.5 us with thirty-two: few long streams per compute
    // unit serve the memory system better than many short ones, and every split adds to the merge
    int n_splits = ctx->opt_attn_splits > 0 ? ctx->opt_attn_splits : (ctx->compute_units + pairs - 1) / pairs;
    if (n_splits > chunks) n_splits = chunks;
    if (n_splits > kMaxSplits) n_splits = kMaxSplits;
    return n_splits < 1 ? 1 : n_splits;
}

// Allocates zeroed split counters; shared with the decoder, which owns its own.
int skn_attn_alloc_counters(skn_ctx* ctx, int n_pairs, int** out) {
    *out = nullptr;
    hipError_t e = hipMalloc((void**)out, (size_t)n_pairs * sizeof(int));
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return skn_fail(ctx, SKN_ERR_OOM, "attention split counters (%d): %s", n_pairs, hipGetErrorString(e));
    }
    SKN_HIP(ctx, hipMemsetAsync(*out, 0, (size_t)n_pairs * sizeof(int), ctx->stream));
    return SKN_OK;
}

// ---- the entry point that allocates nothing ---------------------------------------------------------------
// Split partials and split counters of skn_attn_decode_static live in one file-scope device array instead of
// memory from hipMalloc.  `attn_static_scratch` below is the host-side stand-in of that array: only the address
// hipGetSymbolAddress returns for it (kept per device in g_static_scratch) is ever handed to a kernel.
namespace {
constexpr int kStaticPairs = 4096;                                   // (sequence, head) pairs: one counter each
constexpr size_t kStaticPartialBytes = (size_t)4 << 20;              // partials: pairs * splits * (head_dim + 2) floats
constexpr size_t kStaticCounterBytes = (size_t)kStaticPairs * sizeof(int);
constexpr int kMaxDevices = 64;
__device__ __align__(256) unsigned char attn_static_scratch[kStaticPartialBytes + kStaticCounterBytes];
unsigned char* g_static_scratch[kMaxDevices] = {};  // device address of the array, per device

__global__ void attn_clear_counters_kernel(int* counters, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) counters[i] = 0;
}
}  // namespace

// Called by skn_init with the context's device current.
int skn_attn_init(skn_ctx* ctx) {
    SKN_REQUIRE(ctx, ctx->device >= 0 && ctx->device < kMaxDevices, SKN_ERR_ARG, "device index %d is beyond %d", ctx->device,
                kMaxDevices);
    if (!g_static_scratch[ctx->device]) {
        void* p = nullptr;
        SKN_HIP(ctx, hipGetSymbolAddress(&p, HIP_SYMBOL(attn_static_scratch)));
        SKN_REQUIRE(ctx, p != nullptr, SKN_ERR_HIP, "hipGetSymbolAddress returned no address for the attention scratch");
        g_static_scratch[ctx->device] = static_cast<unsigned char*>(p);
    }
    return SKN_OK;
}

extern "C" int skn_attn_decode_static(skn_ctx* ctx, skn_kv* kv, const float* q_dev, float scale, float* out_dev) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_attn_decode_static: ctx is null");
    SKN_REQUIRE(ctx, kv != nullptr, SKN_ERR_ARG, "skn_attn_decode_static: kv is null");
    SKN_REQUIRE(ctx, q_dev && out_dev, SKN_ERR_ARG, "skn_attn_decode_static: null pointer");
    unsigned char* base = g_static_scratch[ctx->device];
    SKN_REQUIRE(ctx, base != nullptr, SKN_ERR_STATE, "skn_attn_decode_static: the scratch array has no address on device %d",
                ctx->device);
    const int pairs = kv->n_seq * kv->n_head;
    SKN_REQUIRE(ctx, pairs <= kStaticPairs, SKN_ERR_SHAPE,
                "skn_attn_decode_static: %d (sequence, head) pairs exceed the static scratch (at most %d)", pairs, kStaticPairs);
    int max_ctx = 0;
    for (int s = 0; s < kv->n_seq; s++)
        if (kv->len[s] > max_ctx) max_ctx = kv->len[s];
    const int n_splits = skn_attn_splits(ctx, pairs, max_ctx);
    const size_t need = (size_t)pairs * n_splits * (kv->head_dim + 2) * sizeof(float);
    SKN_REQUIRE(ctx, n_splits == 1 || need <= kStaticPartialBytes, SKN_ERR_SHAPE,
                "skn_attn_decode_static: %d pairs x %d splits x head_dim %d need %zu bytes of partials (at most %zu)", pairs,
                n_splits, kv->head_dim, need, kStaticPartialBytes);
    float* partial = reinterpret_cast<float*>(base);
    int* counters = reinterpret_cast<int*>(base + kStaticPartialBytes);
    // the array keeps what the last call left (a call that was cut short may have left counts): start from zero
    skn_launch(ctx, attn_clear_counters_kernel, dim3((pairs + 255) / 256), dim3(256), 0, counters, pairs);
    SKN_LAUNCH_CHECK(ctx);
    return skn_attn_launch_ex(ctx, kv, q_dev, kv->len_dev, kv->n_seq, -1, n_splits, partial, counters, scale, out_dev);
}

int skn_attn_launch(skn_ctx* ctx, skn_kv* kv, const float* q_dev, const int32_t* nctx_dev, int max_ctx, float scale,
                    float* out_dev) {
    const int D = kv->head_dim;
    const int pairs = kv->n_seq * kv->n_head;
    const int n_splits = skn_attn_splits(ctx, pairs, max_ctx);
    const size_t need = (size_t)pairs * n_splits * (D + 2) * sizeof(float);
    if (need > ctx->attn_scratch_bytes) {
        SKN_HIP(ctx, hipStreamSynchronize(ctx->stream));
        if (ctx->attn_scratch) SKN_HIP(ctx, hipFree(ctx->attn_scratch));
        ctx->attn_scratch = nullptr;
        ctx->attn_scratch_bytes = 0;
        const size_t grow = need < (1u << 20) ? (1u << 20) : need;
        hipError_t e = hipMalloc(&ctx->attn_scratch, grow);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return skn_fail(ctx, SKN_ERR_OOM, "skn_attn_decode: %zu bytes of scratch: %s", grow, hipGetErrorString(e));
        }
        ctx->attn_scratch_bytes = grow;
    }
    if (pairs > ctx->attn_counters_cap) {
        SKN_HIP(ctx, hipStreamSynchronize(ctx->stream));
        if (ctx->attn_counters) SKN_HIP(ctx, hipFree(ctx->attn_counters));
        ctx->attn_counters = nullptr;
        ctx->attn_counters_cap = 0;
        const int cap = pairs < 1024 ? 1024 : pairs;
        const int rc = skn_attn_alloc_counters(ctx, cap, &ctx->attn_counters);
        if (rc != SKN_OK) return rc;
        ctx->attn_counters_cap = cap;
    }
    return skn_attn_launch_ex(ctx, kv, q_dev, nctx_dev, kv->n_seq, -1, n_splits, (float*)ctx->attn_scratch,
                              ctx->attn_counters, scale, out_dev);
}

extern "C" int skn_attn_decode(skn_ctx* ctx, skn_kv* kv, const float* q_dev, const int32_t* n_ctx_host, float scale,
                               float* out_dev) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_attn_decode: ctx is null");
    SKN_REQUIRE(ctx, kv != nullptr, SKN_ERR_ARG, "skn_attn_decode: kv is null");
    SKN_REQUIRE(ctx, q_dev && out_dev, SKN_ERR_ARG, "skn_attn_decode: null pointer");
    int max_ctx = 0;
    const int32_t* nctx_dev = kv->len_dev;
    if (n_ctx_host) {
        for (int s = 0; s < kv->n_seq; s++) {
            SKN_REQUIRE(ctx, n_ctx_host[s] >= 0 && n_ctx_host[s] <= kv->len[s], SKN_ERR_RANGE,
                        "skn_attn_decode: %d tokens requested of sequence %d holding %d", n_ctx_host[s], s, kv->len[s]);
            if (n_ctx_host[s] > max_ctx) max_ctx = n_ctx_host[s];
        }
        kv->nctx_host.assign(n_ctx_host, n_ctx_host + kv->n_seq);
        SKN_HIP(ctx, hipMemcpyAsync(kv->nctx_dev, kv->nctx_host.data(), (size_t)kv->n_seq * sizeof(int32_t),
                                    hipMemcpyHostToDevice, ctx->stream));
        nctx_dev = kv->nctx_dev;
    } else {
        for (int s = 0; s < kv->n_seq; s++)
            if (kv->len[s] > max_ctx) max_ctx = kv->len[s];
    }
    return skn_attn_launch(ctx, kv, q_dev, nctx_dev, max_ctx, scale, out_dev);
}
