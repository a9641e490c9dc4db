// Causal attention of many query rows of one sequence (prompt processing) on the matrix cores.
//
//   out[t, h, :] = softmax(q[t, h, :] . K[0 : n_t, h, :]^T * scale) . V[0 : n_t, h, :],   n_t = first_ctx + t
//
// Two launches.  (1) attn_frag_kernel copies the K and V rows of the sequence out of the paged cache into the
// order in which the matrix instructions take them: per head and tile of 32 tokens, the 64 lanes x 16 bytes of
// every operand are contiguous (K as the row operand of K . Q^T, V transposed as the row operand of V^T . P^T),
// so the attention kernel loads an operand with one coalesced 1 KiB load and uses neither LDS nor barriers.
// (2) attn_prefill_kernel: one workgroup of four wavefronts per (32 query rows, head); wavefront w walks the key
// tiles w, w + 4, ... up to the causal limit with the online softmax, and the four partial results are merged
// through LDS: S^T = K Q^T (scores of a query sit in one lane column: its maximum and sum need no
// cross-lane traffic beyond the two lane halves), P = exp2(S - max), O^T += V^T P^T.
// Precision: K and V are the cached fp16 values; q (pre-multiplied by scale * log2 e) and P enter as fp16 pairs
// hi + lo (two matrix instructions per step), products and sums are fp32.
#include "kv.h"

namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

// In the accumulator layout of v_mfma_f32_32x32x16_f16, register x of lane l = 32 h + n holds row
// 8 (x / 4) + 4 h + x % 4 of column n.  Registers 0..7 (8..15) of the score tile are handed on as the eight k
// values of lane half h in the first (second) k-step of the next product, so position p of half h in k-step s
// stands for key 16 s + 8 (p / 4) + 4 h + p % 4 of the tile -- the V^T operand is written in that key order.
__device__ __forceinline__ int key_of(int s, int h, int p) { return 16 * s + 8 * (p >> 2) + 4 * h + (p & 3); }

// grid (tiles, heads), 256 threads.  Tokens at or beyond n_tokens are written as zeros.
// kfrag: [head][tile][k-step D/16][lane] x 8 halves: lane 32 h + r = elements 16 s + 8 h .. + 7 of key r.
// vfrag: [head][tile][32-row block of d][k-step 2][lane] x 8 halves: lane 32 h + r = element 32 b + r of the
//        eight keys key_of(s, h, 0..7).
template <int D>
__global__ __launch_bounds__(256) void attn_frag_kernel(const uint16_t* __restrict__ k_pool, const uint16_t* __restrict__ v_pool,
                                                        const int32_t* __restrict__ table, int n_head, int page_tokens,
                                                        int n_tokens, int n_tiles, u32x4* __restrict__ kfrag,
                                                        u32x4* __restrict__ vfrag) {
    constexpr int kPieces = D / 8;             // 16-byte pieces of a row
    constexpr int kPitch = D + 8;              // LDS row pitch in halves
    __shared__ __align__(16) uint16_t vt[32 * kPitch];
    const int tile = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
    u32x4* kout = kfrag + ((size_t)head * n_tiles + tile) * (D / 16) * 64;
    u32x4* vout = vfrag + ((size_t)head * n_tiles + tile) * (D / 16) * 64;
    for (int i = tid; i < 32 * kPieces; i += 256) {
        const int r = i / kPieces, pc = i - r * kPieces;
        const int t = 32 * tile + r;
        u32x4 kk = {0u, 0u, 0u, 0u}, vv = kk;
        if (t < n_tokens) {
            const int page = table[t / page_tokens], slot = t % page_tokens;
            const size_t off = (((size_t)page * n_head + head) * page_tokens + slot) * D + 8 * pc;
            kk = *reinterpret_cast<const u32x4*>(k_pool + off);
            vv = *reinterpret_cast<const u32x4*>(v_pool + off);
        }
        kout[(pc >> 1) * 64 + 32 * (pc & 1) + r] = kk;
        *reinterpret_cast<u32x4*>(vt + r * kPitch + 8 * pc) = vv;
    }
    __syncthreads();
    for (int i = tid; i < (D / 32) * 2 * 64; i += 256) {
        const int lane = i & 63, s = (i >> 6) & 1, b = i >> 7;
        const int h = lane >> 5, r = lane & 31;
        uint32_t w[4];
#pragma unroll
        for (int p = 0; p < 8; p += 2) {
            const uint32_t lo = vt[key_of(s, h, p) * kPitch + 32 * b + r], hi = vt[key_of(s, h, p + 1) * kPitch + 32 * b + r];
            w[p >> 1] = lo | (hi << 16);
        }
        vout[i] = u32x4{w[0], w[1], w[2], w[3]};
    }
}

// grid (query blocks of 32, heads), four wavefronts each; the block with the most keys first.
// q, out: fp32 [n_queries][n_head][D]; query row t attends to keys [0, first_ctx + t).
template <int D>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void attn_prefill_kernel(const float* __restrict__ q, const u32x4* __restrict__ kfrag,
                                                          const u32x4* __restrict__ vfrag, float* __restrict__ out,
                                                          int n_queries, int n_head, int kv_group, int first_ctx, int n_tiles,
                                                          float scale_log2e) {
    constexpr int KS = D / 16, DB = D / 32;
    __shared__ float part[3][DB * 16 + 2][64];  // running maximum, sum and accumulators of wavefronts 1..3
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, h = lane >> 5, n = lane & 31;
    const int qb = (int)gridDim.x - 1 - (int)blockIdx.x, head = blockIdx.y;
    const int t = min(32 * qb + n, n_queries - 1);  // (rows past the end repeat the last one and are not stored)
    const int n_ctx = first_ctx + t;                // keys this lane's query sees
    // the last tile any query of the block needs
    const int last_tile = min((first_ctx + min(32 * qb + 31, n_queries - 1) - 1) >> 5, n_tiles - 1);

    // q as the column operand: lane 32 h + n holds elements 16 s + 8 h .. + 7 of query n, as an fp16 pair
    half8_t qh[KS], ql[KS];
    const float* qr = q + ((size_t)t * n_head + head) * D + 8 * h;
#pragma unroll
    for (int s = 0; s < KS; s++) {
        const float4 a = *reinterpret_cast<const float4*>(qr + 16 * s), b = *reinterpret_cast<const float4*>(qr + 16 * s + 4);
        const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            _Float16 x, y;
            skn_split_hilo(v[i] * scale_log2e, x, y);
            qh[s][i] = x, ql[s][i] = y;
        }
    }
    float16_t o[DB];
#pragma unroll
    for (int b = 0; b < DB; b++)
#pragma unroll
        for (int x = 0; x < 16; x++) o[b][x] = 0.f;
    float mrun = -INFINITY, lrun = 0.f;  // running maximum (both halves agree) and this half's share of the sum

    // (grouped queries: kv_group consecutive query heads read the keys and values of one cached head)
    const u32x4* kp = kfrag + (size_t)(head / kv_group) * n_tiles * KS * 64 + lane;
    const u32x4* vp = vfrag + (size_t)(head / kv_group) * n_tiles * KS * 64 + lane;
    u32x4 kf[KS];
#pragma unroll
    for (int s = 0; s < KS; s++) kf[s] = kp[((size_t)min(wave, last_tile) * KS + s) * 64];
    for (int tile = wave; tile <= last_tile; tile += 4) {
        u32x4 vf[KS];
#pragma unroll
        for (int s = 0; s < KS; s++) vf[s] = vp[((size_t)tile * KS + s) * 64];
        // S^T = K Q^T: rows = keys of the tile, column = this lane's query (in units of log2 e)
        float16_t sc;
#pragma unroll
        for (int x = 0; x < 16; x++) sc[x] = 0.f;
#pragma unroll
        for (int s = 0; s < KS; s++) {
            const half8_t a = __builtin_bit_cast(half8_t, kf[s]);
            sc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qh[s], sc, 0, 0, 0);
            sc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, ql[s], sc, 0, 0, 0);
        }
        // the next tile's keys (past the end: the last tile again, unused)
        const int nt = min(tile + 4, last_tile);
#pragma unroll
        for (int s = 0; s < KS; s++) kf[s] = kp[((size_t)nt * KS + s) * 64];
        // causal mask and the tile maximum of this query
        float mt = -INFINITY;
#pragma unroll
        for (int x = 0; x < 16; x++) {
            const int key = 32 * tile + 8 * (x >> 2) + 4 * h + (x & 3);
            sc[x] = key < n_ctx ? sc[x] : -INFINITY;
            mt = fmaxf(mt, sc[x]);
        }
        mt = fmaxf(mt, __shfl_xor(mt, 32));
        const float mnew = fmaxf(mrun, mt);
        // (a wavefront that has not met a visible key of this query yet: everything stays zero)
        const float alpha = mnew == -INFINITY ? 1.f : exp2f(mrun - mnew);
        mrun = mnew;
        float psum = 0.f;
        half8_t ph[2], pl[2];
#pragma unroll
        for (int x = 0; x < 16; x++) {
            const float p = mnew == -INFINITY ? 0.f : exp2f(sc[x] - mnew);
            psum += p;
            _Float16 a, b;
            skn_split_hilo(p, a, b);
            ph[x >> 3][x & 7] = a, pl[x >> 3][x & 7] = b;
        }
        lrun = lrun * alpha + psum;
        if (__any(alpha != 1.f)) {
#pragma unroll
            for (int b = 0; b < DB; b++)
#pragma unroll
                for (int x = 0; x < 16; x++) o[b][x] *= alpha;
        }
        // O^T += V^T P^T: rows = elements of the head, column = this lane's query
#pragma unroll
        for (int b = 0; b < DB; b++)
#pragma unroll
            for (int s = 0; s < 2; s++) {
                const half8_t a = __builtin_bit_cast(half8_t, vf[2 * b + s]);
                o[b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, ph[s], o[b], 0, 0, 0);
                o[b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pl[s], o[b], 0, 0, 0);
            }
    }
    // merge: wavefronts 1..3 hand their state to wavefront 0 (which owns tile 0, where key 0 is visible to every
    // query: its maximum is finite)
    if (wave > 0) {
        part[wave - 1][0][lane] = mrun;
        part[wave - 1][1][lane] = lrun;
#pragma unroll
        for (int b = 0; b < DB; b++)
#pragma unroll
            for (int x = 0; x < 16; x++) part[wave - 1][2 + 16 * b + x][lane] = o[b][x];
    }
    __syncthreads();
    if (wave > 0) return;
    {
        float mall = mrun;
#pragma unroll
        for (int w = 0; w < 3; w++) mall = fmaxf(mall, part[w][0][lane]);
        const float f0 = exp2f(mrun - mall);
        lrun *= f0;
#pragma unroll
        for (int b = 0; b < DB; b++)
#pragma unroll
            for (int x = 0; x < 16; x++) o[b][x] *= f0;
#pragma unroll
        for (int w = 0; w < 3; w++) {
            const float mw = part[w][0][lane];
            const float f = mw == -INFINITY ? 0.f : exp2f(mw - mall);
            lrun += part[w][1][lane] * f;
#pragma unroll
            for (int b = 0; b < DB; b++)
#pragma unroll
                for (int x = 0; x < 16; x++) o[b][x] += part[w][2 + 16 * b + x][lane] * f;
        }
    }
    const float ltot = lrun + __shfl_xor(lrun, 32);
    const float inv = ltot > 0.f ? 1.0f / ltot : 0.f;
    if (32 * qb + n < n_queries) {
        float* orow = out + ((size_t)t * n_head + head) * D + 4 * h;
#pragma unroll
        for (int b = 0; b < DB; b++)
#pragma unroll
            for (int g = 0; g < 4; g++)
                *reinterpret_cast<float4*>(orow + 32 * b + 8 * g) =
                    make_float4(o[b][4 * g] * inv, o[b][4 * g + 1] * inv, o[b][4 * g + 2] * inv, o[b][4 * g + 3] * inv);
    }
}

template <int D>
int launch_prefill(skn_ctx* ctx, skn_kv* kv, int seq, const float* q_dev, int n_queries, int first_ctx, float scale,
                   float* out_dev, int n_q_head) {
    const int n_tokens = first_ctx + n_queries - 1;  // keys the last query sees
    const int n_tiles = (n_tokens + 31) / 32;
    const size_t frag_bytes = (size_t)kv->n_head * n_tiles * 32 * D * 2;
    if (2 * frag_bytes > ctx->prefill_ws_bytes) {
        SKN_HIP(ctx, hipStreamSynchronize(ctx->stream));
        if (ctx->prefill_ws) SKN_HIP(ctx, hipFree(ctx->prefill_ws));
        ctx->prefill_ws = nullptr;
        ctx->prefill_ws_bytes = 0;
        hipError_t e = hipMalloc(&ctx->prefill_ws, 2 * frag_bytes);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return skn_fail(ctx, SKN_ERR_OOM, "skn_attn_prefill: %zu bytes of workspace: %s", 2 * frag_bytes, hipGetErrorString(e));
        }
        ctx->prefill_ws_bytes = 2 * frag_bytes;
    }
    u32x4* kfrag = (u32x4*)ctx->prefill_ws;
    u32x4* vfrag = (u32x4*)((uint8_t*)ctx->prefill_ws + frag_bytes);
    skn_launch(ctx, attn_frag_kernel<D>, dim3(n_tiles, kv->n_head), dim3(256), 0, (const uint16_t*)kv->k_pool,
               (const uint16_t*)kv->v_pool, (const int32_t*)(kv->page_table_dev + (size_t)seq * kv->pages_per_seq), kv->n_head,
               kv->page_tokens, n_tokens, n_tiles, kfrag, vfrag);
    SKN_LAUNCH_CHECK(ctx);
    skn_launch(ctx, attn_prefill_kernel<D>, dim3((n_queries + 31) / 32, n_q_head), dim3(256), 0, q_dev, (const u32x4*)kfrag,
               (const u32x4*)vfrag, out_dev, n_queries, n_q_head, n_q_head / kv->n_head, first_ctx, n_tiles,
               scale * 1.4426950408889634f);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

}  // namespace

// Shared with the decoder.  Query row t of n_queries attends to the first first_ctx + t tokens of sequence seq
// (first_ctx >= 1; all of them must be cached).  head_dim 64 or 128.
int skn_attn_prefill_launch(skn_ctx* ctx, skn_kv* kv, int seq, const float* q_dev, int n_queries, int first_ctx, float scale,
                            float* out_dev, int n_q_head) {
    if (n_q_head <= 0) n_q_head = kv->n_head;
    SKN_REQUIRE(ctx, n_q_head % kv->n_head == 0, SKN_ERR_SHAPE,
                "attention: %d query heads are not a multiple of the %d cached heads", n_q_head, kv->n_head);
    if (kv->head_dim == 64) return launch_prefill<64>(ctx, kv, seq, q_dev, n_queries, first_ctx, scale, out_dev, n_q_head);
    if (kv->head_dim == 128) return launch_prefill<128>(ctx, kv, seq, q_dev, n_queries, first_ctx, scale, out_dev, n_q_head);
    return skn_fail(ctx, SKN_ERR_SHAPE, "skn_attn_prefill: head_dim %d is not supported (64 or 128)", kv->head_dim);
}

extern "C" int skn_attn_prefill(skn_ctx* ctx, skn_kv* kv, int seq, const float* q_dev, int n_queries, float scale,
                                float* out_dev) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_attn_prefill: ctx is null");
    SKN_REQUIRE(ctx, kv != nullptr, SKN_ERR_ARG, "skn_attn_prefill: kv is null");
    SKN_REQUIRE(ctx, seq >= 0 && seq < kv->n_seq, SKN_ERR_RANGE, "skn_attn_prefill: sequence %d of %d", seq, kv->n_seq);
    SKN_REQUIRE(ctx, n_queries >= 0 && n_queries <= kv->len[seq], SKN_ERR_RANGE,
                "skn_attn_prefill: %d query rows for a sequence holding %d tokens", n_queries, kv->len[seq]);
    if (n_queries == 0) return SKN_OK;
    SKN_REQUIRE(ctx, q_dev && out_dev, SKN_ERR_ARG, "skn_attn_prefill: null pointer");
    SKN_REQUIRE(ctx, ((uintptr_t)q_dev & 15) == 0 && ((uintptr_t)out_dev & 15) == 0, SKN_ERR_ARG,
                "skn_attn_prefill: q and out must be 16-byte aligned");
    return skn_attn_prefill_launch(ctx, kv, seq, q_dev, n_queries, kv->len[seq] - n_queries + 1, scale, out_dev);
}
