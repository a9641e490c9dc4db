// Decode attention over the paged KV cache: out[s,h,:] = softmax(q[s,h,:] . K^T * scale) . V.
//
// One query row per (sequence, head), so every K and V byte is used exactly once: the kernel is an HBM
// stream of 2 * n_ctx * head_dim * 2 bytes per (sequence, head) at 1 flop per byte.  The context is split
// across workgroups (flash-decoding): grid = (splits, heads, sequences); each workgroup walks its token
// range in 64-token tiles, stages the K and V tiles through LDS with 128-bit loads, keeps a running
// (max, sum, output) triple, and writes one partial; a small second kernel merges the partials.
#include "kv.h"

namespace {

constexpr int kTile = 64;

template <int D>
__global__ __launch_bounds__(256) void attn_decode_split_kernel(
    const uint16_t* __restrict__ k_pool, const uint16_t* __restrict__ v_pool, const int32_t* __restrict__ table,
    const int32_t* __restrict__ nctx, const float* __restrict__ q, float* __restrict__ partial, int n_head,
    int page_tokens, int pages_per_seq, int n_splits, float scale, int seq_fixed) {
    constexpr int KROW = D + 8;   // halves per K row in LDS: 16 bytes of padding spread the rows over the banks
    constexpr int CH = D / 8;     // 16-byte chunks per row
    constexpr int QS = D / 4;     // dims per score thread
    constexpr int VEC = D / 64;   // dims per output lane
    __shared__ __align__(16) uint16_t ks[kTile * KROW];
    __shared__ __align__(16) uint16_t vs[kTile * D];
    __shared__ float ps[kTile];
    __shared__ float red_max[4], red_sum[4];
    __shared__ float obuf[4][D];

    // blockIdx.z is the query row: its own sequence by default, or one shared sequence (seq_fixed >= 0) when
    // several query rows attend to prefixes of the same cache (prompt processing)
    const int split = blockIdx.x, h = blockIdx.y, s = blockIdx.z;
    const int kv_seq = seq_fixed >= 0 ? seq_fixed : s;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = nctx[s];
    const int tiles_total = (n + kTile - 1) / kTile;
    const int tiles_per_split = (tiles_total + n_splits - 1) / n_splits;
    const int t_begin = split * tiles_per_split * kTile;
    const int t_end = min(n, t_begin + tiles_per_split * kTile);

    const int tt = tid >> 2, sl = tid & 3;  // score phase: token of the tile, quarter of the head dimension
    float qr[QS];
    {
        const float* qp = q + ((size_t)s * n_head + h) * D + sl * QS;
#pragma unroll
        for (int i = 0; i < QS; i++) qr[i] = qp[i] * scale;
    }
    float o[VEC];
#pragma unroll
    for (int v = 0; v < VEC; v++) o[v] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;
    const int32_t* trow = table + (size_t)kv_seq * pages_per_seq;

    for (int t0 = t_begin; t0 < t_end; t0 += kTile) {
        const int nt = min(kTile, t_end - t0);
        for (int idx = tid; idx < kTile * CH; idx += 256) {
            const int r = idx / CH, c = idx % CH;
            uint4 kk = make_uint4(0, 0, 0, 0), vv = kk;
            if (r < nt) {
                const int t = t0 + r;
                const int page = trow[t / page_tokens];
                const size_t off = (((size_t)page * n_head + h) * page_tokens + (t % page_tokens)) * D + c * 8;
                kk = *reinterpret_cast<const uint4*>(k_pool + off);
                vv = *reinterpret_cast<const uint4*>(v_pool + off);
            }
            *reinterpret_cast<uint4*>(ks + r * KROW + c * 8) = kk;
            *reinterpret_cast<uint4*>(vs + r * D + c * 8) = vv;
        }
        __syncthreads();

        // scores: four lanes per token, each over a quarter of the head dimension
        float sc = 0.f;
        {
            const uint16_t* kr = ks + tt * KROW + sl * QS;
#pragma unroll
            for (int i = 0; i < QS; i += 8) {
                const uint4 u = *reinterpret_cast<const uint4*>(kr + i);
                const uint32_t wds[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    sc = fmaf(h2f_bits(wds[j] & 0xFFFF), qr[i + 2 * j], sc);
                    sc = fmaf(h2f_bits(wds[j] >> 16), qr[i + 2 * j + 1], sc);
                }
            }
        }
        sc += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(sc), 0xB1, 0xF, 0xF, true));
        sc += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(sc), 0x4E, 0xF, 0xF, true));
        if (tt >= nt) sc = -INFINITY;
        const float wmax = wave_max(sc);
        if (lane == 0) red_max[wave] = wmax;
        __syncthreads();
        const float tile_max = fmaxf(fmaxf(red_max[0], red_max[1]), fmaxf(red_max[2], red_max[3]));
        const float m_new = fmaxf(m_run, tile_max);
        const float p = (tt < nt) ? __expf(sc - m_new) : 0.f;
        if (sl == 0) ps[tt] = p;
        const float wsum = wave_sum(sl == 0 ? p : 0.f);
        if (lane == 0) red_sum[wave] = wsum;
        const float alpha = __expf(m_run - m_new);  // 0 on the first tile (m_run = -inf)
        __syncthreads();
        l_run = l_run * alpha + ((red_sum[0] + red_sum[1]) + (red_sum[2] + red_sum[3]));
        m_run = m_new;

        // output: wave w takes tokens 16w..16w+15 of the tile, lane l the dims VEC*l..
#pragma unroll
        for (int v = 0; v < VEC; v++) o[v] *= alpha;
#pragma unroll 4
        for (int j = 0; j < 16; j++) {
            const int t = wave * 16 + j;
            const float pj = ps[t];
            const uint16_t* vr = vs + t * D + lane * VEC;
            if constexpr (VEC == 1) {
                o[0] = fmaf(pj, h2f_bits(vr[0]), o[0]);
            } else if constexpr (VEC == 2) {
                const uint32_t u = *reinterpret_cast<const uint32_t*>(vr);
                o[0] = fmaf(pj, h2f_bits(u & 0xFFFF), o[0]);
                o[1] = fmaf(pj, h2f_bits(u >> 16), o[1]);
            } else {
                const uint2 u = *reinterpret_cast<const uint2*>(vr);
                o[0] = fmaf(pj, h2f_bits(u.x & 0xFFFF), o[0]);
                o[1] = fmaf(pj, h2f_bits(u.x >> 16), o[1]);
                o[2] = fmaf(pj, h2f_bits(u.y & 0xFFFF), o[2]);
                o[3] = fmaf(pj, h2f_bits(u.y >> 16), o[3]);
            }
        }
        __syncthreads();  // the next tile overwrites ks / vs / ps
    }

#pragma unroll
    for (int v = 0; v < VEC; v++) obuf[wave][lane * VEC + v] = o[v];
    __syncthreads();
    float* dst = partial + (((size_t)s * n_head + h) * n_splits + split) * (D + 2);
    if (tid < D) dst[tid] = (obuf[0][tid] + obuf[1][tid]) + (obuf[2][tid] + obuf[3][tid]);
    if (tid == 0) {
        dst[D] = m_run;
        dst[D + 1] = l_run;
    }
}

// grid = sequences * heads, block = head_dim threads
__global__ void attn_merge_kernel(const float* __restrict__ partial, float* __restrict__ out, int n_splits, int D) {
    const float* base = partial + (size_t)blockIdx.x * n_splits * (D + 2);
    const int d = threadIdx.x;
    float M = -INFINITY;
    for (int i = 0; i < n_splits; i++) M = fmaxf(M, base[i * (D + 2) + D]);
    float acc = 0.f, L = 0.f;
    for (int i = 0; i < n_splits; i++) {
        const float mi = base[i * (D + 2) + D];
        const float wgt = (mi == -INFINITY) ? 0.f : __expf(mi - M);
        L = fmaf(wgt, base[i * (D + 2) + D + 1], L);
        acc = fmaf(wgt, base[i * (D + 2) + d], acc);
    }
    out[(size_t)blockIdx.x * D + d] = L > 0.f ? acc / L : 0.f;
}

}  // namespace

// Shared with the decoder.  n_queries query rows; row z attends to nctx_dev[z] tokens of sequence z
// (seq_fixed < 0) or of sequence seq_fixed.  `partial` must hold n_queries * n_head * n_splits * (D + 2) floats.
int skn_attn_launch_ex(skn_ctx* ctx, skn_kv* kv, const float* q_dev, const int32_t* nctx_dev, int n_queries,
                       int seq_fixed, int n_splits, float* partial, float scale, float* out_dev) {
    const int D = kv->head_dim;
    SKN_REQUIRE(ctx, D == 64 || D == 128 || D == 256, SKN_ERR_SHAPE,
                "skn_attn_decode: head_dim %d is not supported (64, 128 or 256)", D);
    dim3 grid(n_splits, kv->n_head, n_queries), block(256);
#define SKN_ATTN_LAUNCH(DD)                                                                                        \
    skn_launch(ctx, attn_decode_split_kernel<DD>, grid, block, 0, kv->k_pool, kv->v_pool, kv->page_table_dev,     \
               nctx_dev, q_dev, partial, kv->n_head, kv->page_tokens, kv->pages_per_seq, n_splits, scale, seq_fixed)
    if (D == 64) SKN_ATTN_LAUNCH(64);
    else if (D == 128) SKN_ATTN_LAUNCH(128);
    else SKN_ATTN_LAUNCH(256);
#undef SKN_ATTN_LAUNCH
    SKN_LAUNCH_CHECK(ctx);
    skn_launch(ctx, attn_merge_kernel, dim3(n_queries * kv->n_head), dim3(D), 0, (const float*)partial, out_dev,
               n_splits, D);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

int skn_attn_splits(skn_ctx* ctx, int pairs, int max_ctx) {
    const int tiles = (max_ctx + kTile - 1) / kTile;
    int n_splits = ctx->opt_attn_splits > 0 ? ctx->opt_attn_splits : (4 * ctx->compute_units + pairs - 1) / pairs;
    if (n_splits > tiles) n_splits = tiles;
    return n_splits < 1 ? 1 : n_splits;
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
    return skn_attn_launch_ex(ctx, kv, q_dev, nctx_dev, kv->n_seq, -1, n_splits, (float*)ctx->attn_scratch, scale,
                              out_dev);
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
