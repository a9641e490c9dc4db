// Llama-style decoder over the quantized kernels: batched prompt processing (GEMM) and greedy decode (matvec)
// for one sequence.  Per layer:  x += Wo . attn(rope(Wq xn), cache(rope(Wk xn), Wv xn)),  xn = rmsnorm(x);
// x += Wdown . (silu(Wgate xn) * (Wup xn)).  Logits = Whead . rmsnorm(x).
//
// A decode step reads every scalar that changes from step to step (token id, position, context length, step
// index) from device memory, so that one captured HIP graph of the ~480 kernel launches of a step can be
// replayed for every token.  The graph holds kernels only (no memset / memcpy nodes).
#include "kv.h"
#include "gemm_q6k.h"

#include <algorithm>
#include <cmath>

struct skn_llama {
    skn_llama_config cfg;
    skn_llama_weights w;
    std::vector<skn_llama_layer> layers;
    std::vector<skn_kv*> kv;  // one single-sequence cache per layer
    // decode-step buffers
    float *x = nullptr, *xn = nullptr, *q = nullptr, *k = nullptr, *v = nullptr, *att = nullptr, *proj = nullptr;
    float *gate = nullptr, *up = nullptr, *mid = nullptr, *logits = nullptr, *attn_partial = nullptr;
    int *attn_counters = nullptr, *pcounters = nullptr;  // split counters of the attention launches (zero between launches)
    int32_t* state = nullptr;       // [0] token, [1] position, [2] context length, [3] step index
    int32_t* tokens_out = nullptr;  // device array of produced tokens
    double* inv_freq = nullptr;     // rope_base^(-2i / head_dim), i < head_dim / 2, formed in double on the host
    int tokens_cap = 0;
    int pos = 0;                    // host mirror of the position
    // prompt buffers (grown to the longest prompt seen)
    int prompt_cap = 0;
    float *px = nullptr, *pxn = nullptr, *pq = nullptr, *pk = nullptr, *pv = nullptr, *patt = nullptr, *pproj = nullptr;
    float *pgate = nullptr, *pup = nullptr, *pmid = nullptr, *ppartial = nullptr;
    uint16_t *pb16 = nullptr, *pk16 = nullptr, *pv16 = nullptr;
    int32_t *ptok = nullptr, *pnctx = nullptr;
    // captured decode step
    hipGraph_t graph = nullptr;
    hipGraphExec_t graph_exec = nullptr;
    int graph_splits = 0;
    int graph_generation = -1;  // ctx->opt_generation at capture: every option decode_step reads, and the stream
    // fp16-pair copies of the matrices that are not Q4_K, for the prompt GEMMs (made on first use when the option
    // llama.expand_weights is set): seven per layer in the order q, k, v, o, gate, up, down
    std::vector<void*> expanded;
    long long expanded_bytes = 0;
    std::vector<void*> owned;
};

namespace {

// ---- kernels that read their step-dependent scalars from device memory -----------------------------------

// One row of a [vocab, hidden] quantized embedding table -> fp32.  grid = rows to embed, tokens from device.
__global__ __launch_bounds__(1024) void embed_rows_kernel(const uint8_t* __restrict__ table, int type, int hidden,
                                                         const int32_t* __restrict__ tokens, float* __restrict__ out) {
    const int row = blockIdx.x;
    const int tok = tokens[row];
    float* dst = out + (size_t)row * hidden;
    if (type == SKN_TYPE_Q4_K) {
        // four consecutive elements per thread: one sub-block, four consecutive nibble bytes (one aligned dword)
        const uint8_t* src = table + (size_t)tok * (hidden / 256) * 144;
        for (int e = 4 * threadIdx.x; e < hidden; e += 4 * blockDim.x) {
            const uint8_t* b = src + (size_t)(e >> 8) * 144;
            const int i = e & 255, c = i >> 6, r = i & 63, j = 2 * c + (r >= 32);
            const uint4 hdr = *reinterpret_cast<const uint4*>(b);  // d | dmin, scales[0..11]
            const uint32_t w[3] = {hdr.y, hdr.z, hdr.w};
            auto sbyte = [&](int k) { return (w[k >> 2] >> (8 * (k & 3))) & 0xFFu; };
            int sc, m;
            if (j < 4) {
                sc = sbyte(j) & 63;
                m = sbyte(j + 4) & 63;
            } else {
                sc = (sbyte(j + 4) & 0x0F) | ((sbyte(j - 4) >> 6) << 4);
                m = (sbyte(j + 4) >> 4) | ((sbyte(j) >> 6) << 4);
            }
            const uint32_t q4 = *reinterpret_cast<const uint32_t*>(b + 16 + 32 * c + (r & 31));
            const float ds = __fmul_rn(h2f_bits(hdr.x & 0xFFFF), (float)sc);
            const float mm = __fmul_rn(h2f_bits(hdr.x >> 16), (float)m);
            const int sh = (r < 32) ? 0 : 4;
            float4 o;
            o.x = __fsub_rn(__fmul_rn(ds, (float)((q4 >> sh) & 0xF)), mm);
            o.y = __fsub_rn(__fmul_rn(ds, (float)((q4 >> (8 + sh)) & 0xF)), mm);
            o.z = __fsub_rn(__fmul_rn(ds, (float)((q4 >> (16 + sh)) & 0xF)), mm);
            o.w = __fsub_rn(__fmul_rn(ds, (float)((q4 >> (24 + sh)) & 0xF)), mm);
            *reinterpret_cast<float4*>(dst + e) = o;
        }
    } else if (type == SKN_TYPE_Q8_0) {
        const uint8_t* src = table + (size_t)tok * (hidden / 32) * 34;
        for (int e = threadIdx.x; e < hidden; e += blockDim.x) {
            const uint8_t* b = src + (size_t)(e >> 5) * 34;
            dst[e] = __fmul_rn(h2f_bits(load_u16_a2(b)), (float)(int8_t)b[2 + (e & 31)]);
        }
    } else if (type == SKN_TYPE_Q6_K) {
        const uint8_t* src = table + (size_t)tok * (hidden / 256) * 210;
        for (int e = threadIdx.x; e < hidden; e += blockDim.x) {
            const uint8_t* b = src + (size_t)(e >> 8) * 210;
            const int i = e & 255, n = i >> 7, r = i & 127, quarter = r >> 5, l = r & 31;
            uint32_t lo = b[64 * n + l + 32 * (quarter & 1)];
            lo = quarter >= 2 ? lo >> 4 : lo & 0xF;
            const uint32_t hi = (b[128 + 32 * n + l] >> (2 * quarter)) & 3;
            const float sc = (float)(int8_t)b[192 + 8 * n + 2 * quarter + (l >> 4)];
            dst[e] = __fmul_rn(__fmul_rn(h2f_bits(load_u16_a2(b + 208)), sc), (float)((int)(lo | (hi << 4)) - 32));
        }
    } else {  // F32
        const float* src = reinterpret_cast<const float*>(table) + (size_t)tok * hidden;
        for (int e = threadIdx.x; e < hidden; e += blockDim.x) dst[e] = src[e];
    }
}

// Rotary embedding of q and k rows at positions pos0 + row (pos0 from device), then k and v rows go to the
// cache as fp16 at those positions.  grid = (rows, n_head), block = head_dim / 2 threads (one pair each); q has
// n_head heads per row, k and v kv_heads (the first kv_heads blocks of a row handle them).
__global__ void rope_store_kernel(float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v,
                                  uint16_t* __restrict__ k_pool, uint16_t* __restrict__ v_pool,
                                  const int32_t* __restrict__ table, const int32_t* __restrict__ pos0_dev, int n_head,
                                  int kv_heads, int head_dim, int page_tokens, double log2_base) {
    const int row = blockIdx.x, h = blockIdx.y, i = threadIdx.x;
    const int pos = pos0_dev[0] + row;
    float sn, cs;
    skn_rope_sincos(pos, 2 * i, head_dim, log2_base, &sn, &cs);
    const size_t qbase = ((size_t)row * n_head + h) * head_dim + 2 * i;
    const float qa = q[qbase], qb = q[qbase + 1];
    q[qbase] = qa * cs - qb * sn;
    q[qbase + 1] = qa * sn + qb * cs;
    if (h >= kv_heads) return;
    const size_t base = ((size_t)row * kv_heads + h) * head_dim + 2 * i;
    const float ka = k[base], kb = k[base + 1];
    const float k0 = ka * cs - kb * sn, k1 = ka * sn + kb * cs;
    const int page = table[pos / page_tokens];
    const size_t dst = (((size_t)page * kv_heads + h) * page_tokens + (pos % page_tokens)) * head_dim + 2 * i;
    const uint32_t kk = (uint32_t)__half_as_ushort(__float2half_rn(k0)) | ((uint32_t)__half_as_ushort(__float2half_rn(k1)) << 16);
    const uint32_t vv = (uint32_t)__half_as_ushort(__float2half_rn(v[base])) |
                        ((uint32_t)__half_as_ushort(__float2half_rn(v[base + 1])) << 16);
    *reinterpret_cast<uint32_t*>(k_pool + dst) = kk;
    *reinterpret_cast<uint32_t*>(v_pool + dst) = vv;
}

// grid = rows, block = 256.  Rows of up to 8192 elements (multiple of 4) stay in registers between the two
// passes and all loads are issued before the first use.
__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                           float* __restrict__ y, int n, float eps) {
    __shared__ float red[4];
    const float* xr = x + (size_t)blockIdx.x * n;
    float* yr = y + (size_t)blockIdx.x * n;
    const int tid = threadIdx.x;
    const bool in_regs = (n & 3) == 0 && n <= 8192;
    float4 v[8], g[8];
    float ss = 0.f;
    if (in_regs) {
        const int n4 = n >> 2;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int i = min(tid + 256 * j, n4 - 1);
            v[j] = reinterpret_cast<const float4*>(xr)[i];
            g[j] = reinterpret_cast<const float4*>(w)[i];
        }
#pragma unroll
        for (int j = 0; j < 8; j++)
            if (tid + 256 * j < n4) ss += (v[j].x * v[j].x + v[j].y * v[j].y) + (v[j].z * v[j].z + v[j].w * v[j].w);
    } else {
        for (int i = tid; i < n; i += 256) ss = fmaf(xr[i], xr[i], ss);
    }
    ss = wave_sum(ss);
    if ((tid & 63) == 0) red[tid >> 6] = ss;
    __syncthreads();
    const float r = 1.0f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)n + eps);
    if (in_regs) {
        const int n4 = n >> 2;
#pragma unroll
        for (int j = 0; j < 8; j++)
            if (tid + 256 * j < n4)
                reinterpret_cast<float4*>(yr)[tid + 256 * j] =
                    make_float4(v[j].x * r * g[j].x, v[j].y * r * g[j].y, v[j].z * r * g[j].z, v[j].w * r * g[j].w);
    } else {
        for (int i = tid; i < n; i += 256) yr[i] = xr[i] * r * w[i];
    }
}

__global__ void add_rows_kernel(float* __restrict__ y, const float* __restrict__ x, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] += x[i];
}

__global__ void swiglu_rows_kernel(const float* __restrict__ g, const float* __restrict__ u, float* __restrict__ out,
                                   int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const float a = g[i];
        out[i] = a / (1.0f + expf(-a)) * u[i];
    }
}

__global__ void f32_to_bf16_rows_kernel(const float* __restrict__ x, uint16_t* __restrict__ out, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        uint32_t u = __float_as_uint(x[i]);
        if ((u & 0x7FFFFFFFu) > 0x7F800000u) {  // NaN stays NaN (quiet), whatever its payload
            out[i] = (uint16_t)((u >> 16) | 0x40u);
        } else {
            u += 0x7FFFu + ((u >> 16) & 1u);
            out[i] = (uint16_t)(u >> 16);
        }
    }
}

// state = {token, position, context length, step}
__global__ void set_state_kernel(int32_t* state, int token, int pos) {
    if (threadIdx.x == 0) {
        state[0] = token;
        state[1] = pos;
        state[2] = pos + 1;
        state[3] = 0;
    }
}

// single workgroup: argmax of the logits (first maximum) becomes the next token; the step's scalars advance
__global__ __launch_bounds__(1024) void finish_step_kernel(const float* __restrict__ x, int n, int32_t* state,
                                                           int32_t* __restrict__ tokens_out, int advance) {
    __shared__ float bv[16];
    __shared__ int bi[16];
    float best = -INFINITY;
    int besti = 0x7FFFFFFF;
    auto take = [&](float v, int i) {
        if (v > best || (v == best && i < besti)) {
            best = v;
            besti = i;
        }
    };
    // eight float4 per thread and round, all loaded before the first compare
    const int n4 = n >> 2;
    for (int base = 0; base < n4; base += 8 * 1024) {
        float4 v[8];
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = reinterpret_cast<const float4*>(x)[min(base + j * 1024 + (int)threadIdx.x, n4 - 1)];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int i4 = base + j * 1024 + (int)threadIdx.x;
            if (i4 < n4) {
                take(v[j].x, 4 * i4);
                take(v[j].y, 4 * i4 + 1);
                take(v[j].z, 4 * i4 + 2);
                take(v[j].w, 4 * i4 + 3);
            }
        }
    }
    for (int i = 4 * n4 + threadIdx.x; i < n; i += 1024) take(x[i], i);
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
        const int tok = besti == 0x7FFFFFFF ? 0 : besti;
        if (advance) {
            tokens_out[state[3]] = tok;
            state[0] = tok;
            state[1] += 1;
            state[2] += 1;
            state[3] += 1;
        } else {
            tokens_out[0] = tok;
        }
    }
}

__global__ void iota_kernel(int32_t* out, int n, int start) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = start + i;
}

template <typename T>
int dev_alloc(skn_ctx* ctx, skn_llama* m, T** p, size_t count) {
    hipError_t e = hipMalloc((void**)p, count * sizeof(T) < 16 ? 16 : count * sizeof(T));
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return skn_fail(ctx, SKN_ERR_OOM, "skn_llama: %zu bytes: %s", count * sizeof(T), hipGetErrorString(e));
    }
    m->owned.push_back((void*)*p);
    return SKN_OK;
}

unsigned nblk(int64_t n) { return (unsigned)((n + 255) / 256); }

#define SKN_TRY(expr)              \
    do {                           \
        int rc_ = (expr);          \
        if (rc_ != SKN_OK) return rc_; \
    } while (0)

// the launches of one decode step (eagerly or under stream capture)
int decode_step(skn_ctx* ctx, skn_llama* m, int n_splits) {
    const skn_llama_config& c = m->cfg;
    const int H = c.hidden, F = c.ffn, NH = c.n_head, D = c.head_dim, KVH = c.n_kv_head, KVD = KVH * D;
    const float scale = 1.0f / sqrtf((float)D);
    skn_launch(ctx, embed_rows_kernel, dim3(1), dim3(1024), 0, (const uint8_t*)m->w.tok_embd, m->w.type_embd, H,
               (const int32_t*)m->state, m->x);
    SKN_LAUNCH_CHECK(ctx);
    for (int l = 0; l < c.n_layer; l++) {
        const skn_llama_layer& L = m->layers[l];
        skn_kv* kv = m->kv[l];
        // Five launches per layer where the matrices of a group share one of the formats the fused kernels take
        // (Q4_K, Q5_K, Q4_0, Q4_1, Q5_0, Q5_1, IQ4_NL, Q6_K, Q8_0): [norm + q,k,v + rope + cache store], attention, [Wo + residual],
        // [norm + gate,up + SwiGLU], [Wdown + residual].  A group of mixed or other types takes each type's
        // matvec and the row-wise kernels around it.
        const bool fuse = ctx->opt_llama_fused && H <= 16384 && H % 256 == 0;
        // (q, k, v of different fusable formats: one fused launch per format, each with the rows of its matrices only)
        const bool f_qkv = fuse && skn_matvec_fusable(L.type_q) && skn_matvec_fusable(L.type_k) && skn_matvec_fusable(L.type_v);
        const bool f_o = fuse && skn_matvec_fusable(L.type_o);
        const bool f_gu = fuse && skn_matvec_fusable(L.type_gate) && L.type_up == L.type_gate;
        const bool f_down = ctx->opt_llama_fused && F <= 16384 && F % 256 == 0 && skn_matvec_fusable(L.type_down);
        if (f_qkv) {
            skn_rope_epilogue rope;
            rope.pos_dev = m->state + 1;
            rope.page_table = kv->page_table_dev;
            rope.k_pool = kv->k_pool;
            rope.v_pool = kv->v_pool;
            rope.n_head = KVH;  // (heads of the cache)
            rope.head_dim = D;
            rope.page_tokens = kv->page_tokens;
            rope.log2_base = log2((double)c.rope_base);
            rope.inv_freq = m->inv_freq;
            const int types[3] = {L.type_q, L.type_k, L.type_v}, rows[3] = {H, KVD, KVD};
            const uint8_t* mats[3] = {(const uint8_t*)L.wq, (const uint8_t*)L.wk, (const uint8_t*)L.wv};
            bool done[3] = {false, false, false};
            for (int i = 0; i < 3; i++) {
                if (done[i]) continue;
                skn_q4k_segments part = {{nullptr, nullptr, nullptr}, {0, 0, 0}};
                int n_out = 0;
                for (int j = i; j < 3; j++)
                    if (types[j] == types[i]) part.w[j] = mats[j], part.rows[j] = rows[j], n_out += rows[j], done[j] = true;
                SKN_TRY(skn_matvec_q4k_fused(ctx, part, n_out, H, m->x, L.attn_norm, c.rms_eps, m->q, SKN_EPI_ROPE, &rope, types[i]));
            }
        } else {
            skn_launch(ctx, rmsnorm_rows_kernel, dim3(1), dim3(256), 0, (const float*)m->x, L.attn_norm, m->xn, H, c.rms_eps);
            SKN_LAUNCH_CHECK(ctx);
            SKN_TRY(skn_matvec_q(ctx, L.type_q, L.wq, H, H, m->xn, m->q));
            SKN_TRY(skn_matvec_q(ctx, L.type_k, L.wk, KVD, H, m->xn, m->k));
            SKN_TRY(skn_matvec_q(ctx, L.type_v, L.wv, KVD, H, m->xn, m->v));
            skn_launch(ctx, rope_store_kernel, dim3(1, NH), dim3(D / 2), 0, m->q, (const float*)m->k, (const float*)m->v,
                       kv->k_pool, kv->v_pool, (const int32_t*)kv->page_table_dev, (const int32_t*)(m->state + 1), NH, KVH, D,
                       kv->page_tokens, log2((double)c.rope_base));
            SKN_LAUNCH_CHECK(ctx);
        }
        if (f_o && ctx->opt_llama_attn_wide && n_splits * 128 > 32768 / D) {
            // The attention leaves the partials of its splits unmerged and the output projection's staging merges them:
            // no device-wide counter, no store-then-reload chain inside the attention launch.  A workgroup of sixteen
            // wavefronts takes 32768 / head_dim tokens per round of requests, so the splits are counted in those units.
            const int per_round = 32768 / D;
            int wide = 2;  // 2, 4 or 8 (what the merge in the projection's staging is built for)
            while (wide < 8 && wide * per_round < n_splits * 128) wide *= 2;
            if (ctx->opt_llama_attn_wide > 1) wide = std::min(wide, ctx->opt_llama_attn_wide);  // (tuning: 2, 4 or 8 caps the count)
            float* opart = m->attn_partial;
            float* ml = m->attn_partial + (size_t)wide * NH * D;
            SKN_TRY(skn_attn_launch_unmerged(ctx, kv, m->q, m->state + 2, 1, 0, wide, opart, ml, scale, m->att, NH));
            skn_q4k_segments wo = {{(const uint8_t*)L.wo, nullptr, nullptr}, {H, 0, 0}};
            skn_rope_epilogue mg;
            mg.merge_ml = ml;
            mg.merge_splits = wide;
            mg.merge_pairs = NH;
            mg.merge_head_f4 = D / 4;
            SKN_TRY(skn_matvec_q4k_fused(ctx, wo, H, H, opart, nullptr, 0.f, m->x, SKN_EPI_ADD, &mg, L.type_o));
        } else if (f_o) {
            SKN_TRY(skn_attn_launch_ex(ctx, kv, m->q, m->state + 2, 1, 0, n_splits, m->attn_partial, m->attn_counters, scale, m->att, NH));
            skn_q4k_segments wo = {{(const uint8_t*)L.wo, nullptr, nullptr}, {H, 0, 0}};
            SKN_TRY(skn_matvec_q4k_fused(ctx, wo, H, H, m->att, nullptr, 0.f, m->x, SKN_EPI_ADD, nullptr, L.type_o));
        } else {
            SKN_TRY(skn_attn_launch_ex(ctx, kv, m->q, m->state + 2, 1, 0, n_splits, m->attn_partial, m->attn_counters, scale, m->att, NH));
            SKN_TRY(skn_matvec_q(ctx, L.type_o, L.wo, H, H, m->att, m->proj));
            skn_launch(ctx, add_rows_kernel, dim3(nblk(H)), dim3(256), 0, m->x, (const float*)m->proj, (int64_t)H);
            SKN_LAUNCH_CHECK(ctx);
        }
        if (f_gu) {
            skn_q4k_segments gu = {{(const uint8_t*)L.w_gate, (const uint8_t*)L.w_up, nullptr}, {F, F, 0}};
            SKN_TRY(skn_matvec_q4k_fused(ctx, gu, F, H, m->x, L.ffn_norm, c.rms_eps, m->mid, SKN_EPI_SWIGLU, nullptr, L.type_gate));
        } else {
            skn_launch(ctx, rmsnorm_rows_kernel, dim3(1), dim3(256), 0, (const float*)m->x, L.ffn_norm, m->xn, H, c.rms_eps);
            SKN_LAUNCH_CHECK(ctx);
            SKN_TRY(skn_matvec_q(ctx, L.type_gate, L.w_gate, F, H, m->xn, m->gate));
            SKN_TRY(skn_matvec_q(ctx, L.type_up, L.w_up, F, H, m->xn, m->up));
            skn_launch(ctx, swiglu_rows_kernel, dim3(nblk(F)), dim3(256), 0, (const float*)m->gate, (const float*)m->up,
                       m->mid, (int64_t)F);
            SKN_LAUNCH_CHECK(ctx);
        }
        if (f_down) {
            skn_q4k_segments wd = {{(const uint8_t*)L.w_down, nullptr, nullptr}, {H, 0, 0}};
            SKN_TRY(skn_matvec_q4k_fused(ctx, wd, H, F, m->mid, nullptr, 0.f, m->x, SKN_EPI_ADD, nullptr, L.type_down));
        } else {
            SKN_TRY(skn_matvec_q(ctx, L.type_down, L.w_down, H, F, m->mid, m->proj));
            skn_launch(ctx, add_rows_kernel, dim3(nblk(H)), dim3(256), 0, m->x, (const float*)m->proj, (int64_t)H);
            SKN_LAUNCH_CHECK(ctx);
        }
    }
    // (the final norm folded into the head's matvec was measured: the fused kernel's two rows per wavefront cost the
    // 32000-row head more than the norm's launch saves, 30 us against 22 + 4)
    skn_launch(ctx, rmsnorm_rows_kernel, dim3(1), dim3(256), 0, (const float*)m->x, m->w.out_norm, m->xn, H, c.rms_eps);
    SKN_LAUNCH_CHECK(ctx);
    SKN_TRY(skn_matvec_q(ctx, m->w.type_head, m->w.out_head, c.vocab, H, m->xn, m->logits));
    skn_launch(ctx, finish_step_kernel, dim3(1), dim3(1024), 0, (const float*)m->logits, c.vocab, m->state,
               m->tokens_out, 1);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

void drop_graph(skn_llama* m) {
    if (m->graph_exec) (void)hipGraphExecDestroy(m->graph_exec);
    if (m->graph) (void)hipGraphDestroy(m->graph);
    m->graph_exec = nullptr;
    m->graph = nullptr;
    m->graph_splits = 0;
    m->graph_generation = -1;
}

// frees a buffer of the model now (the stream must be idle) and forgets it
template <typename T>
void dev_release(skn_llama* m, T** p) {
    if (!*p) return;
    for (size_t i = 0; i < m->owned.size(); i++)
        if (m->owned[i] == (void*)*p) {
            m->owned.erase(m->owned.begin() + i);
            break;
        }
    (void)hipFree((void*)*p);
    *p = nullptr;
}

int ensure_prompt_buffers(skn_ctx* ctx, skn_llama* m, int T) {
    if (T <= m->prompt_cap) return SKN_OK;
    const skn_llama_config& c = m->cfg;
    const size_t H = c.hidden, F = c.ffn;
    // the buffers of a shorter prompt are released first (nothing on the stream may still read them)
    if (m->prompt_cap > 0) {
        SKN_HIP(ctx, hipStreamSynchronize(ctx->stream));
        dev_release(m, &m->px); dev_release(m, &m->pxn); dev_release(m, &m->pq); dev_release(m, &m->pk);
        dev_release(m, &m->pv); dev_release(m, &m->patt); dev_release(m, &m->pproj); dev_release(m, &m->pgate);
        dev_release(m, &m->pup); dev_release(m, &m->pmid); dev_release(m, &m->pb16); dev_release(m, &m->ptok);
        dev_release(m, &m->pnctx); dev_release(m, &m->ppartial); dev_release(m, &m->pcounters);
        m->prompt_cap = 0;
    }
    SKN_TRY(dev_alloc(ctx, m, &m->px, T * H));
    SKN_TRY(dev_alloc(ctx, m, &m->pxn, T * H));
    SKN_TRY(dev_alloc(ctx, m, &m->pq, T * H));
    SKN_TRY(dev_alloc(ctx, m, &m->pk, T * H));
    SKN_TRY(dev_alloc(ctx, m, &m->pv, T * H));
    SKN_TRY(dev_alloc(ctx, m, &m->patt, T * H));
    SKN_TRY(dev_alloc(ctx, m, &m->pproj, T * H));
    SKN_TRY(dev_alloc(ctx, m, &m->pgate, T * F));
    SKN_TRY(dev_alloc(ctx, m, &m->pup, T * F));
    SKN_TRY(dev_alloc(ctx, m, &m->pmid, T * F));
    SKN_TRY(dev_alloc(ctx, m, &m->pb16, T * (F > H ? F : H)));
    SKN_TRY(dev_alloc(ctx, m, &m->ptok, (size_t)T));
    SKN_TRY(dev_alloc(ctx, m, &m->pnctx, (size_t)T));
    // splits <= ceil(CUs / pairs) keeps pairs * splits below pairs + CUs; the rest is head room
    SKN_TRY(dev_alloc(ctx, m, &m->ppartial, ((size_t)T * c.n_head + 4 * (size_t)ctx->compute_units) * (c.head_dim + 2)));
    SKN_TRY(dev_alloc(ctx, m, &m->pcounters, (size_t)T * c.n_head));
    SKN_HIP(ctx, hipMemsetAsync(m->pcounters, 0, (size_t)T * c.n_head * sizeof(int), ctx->stream));
    m->prompt_cap = T;
    return SKN_OK;
}

int to_bf16(skn_ctx* ctx, const float* x, uint16_t* out, int64_t n) {
    skn_launch(ctx, f32_to_bf16_rows_kernel, dim3(nblk(n)), dim3(256), 0, x, out, n);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

}  // namespace

extern "C" {

int skn_llama_create(skn_ctx* ctx, const skn_llama_config* cfg, const skn_llama_weights* w, skn_llama** out) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_llama_create: ctx is null");
    SKN_REQUIRE(ctx, cfg && w && out, SKN_ERR_ARG, "skn_llama_create: null pointer");
    *out = nullptr;
    SKN_REQUIRE(ctx, cfg->n_layer > 0 && cfg->hidden > 0 && cfg->ffn > 0 && cfg->n_head > 0 && cfg->head_dim > 0 &&
                         cfg->vocab > 0 && cfg->max_tokens > 0 && cfg->page_tokens > 0,
                SKN_ERR_ARG, "skn_llama_create: sizes must be positive");
    SKN_REQUIRE(ctx, cfg->n_kv_head >= 0 && (cfg->n_kv_head == 0 || cfg->n_head % cfg->n_kv_head == 0), SKN_ERR_SHAPE,
                "skn_llama_create: n_kv_head (%d) must divide n_head (%d)", cfg->n_kv_head, cfg->n_head);
    SKN_REQUIRE(ctx, cfg->n_head * cfg->head_dim == cfg->hidden, SKN_ERR_SHAPE,
                "skn_llama_create: n_head * head_dim (%d) must equal hidden (%d)", cfg->n_head * cfg->head_dim,
                cfg->hidden);
    SKN_REQUIRE(ctx, cfg->head_dim == 64 || cfg->head_dim == 128 || cfg->head_dim == 256, SKN_ERR_SHAPE,
                "skn_llama_create: head_dim %d is not supported (64, 128 or 256)", cfg->head_dim);
    SKN_REQUIRE(ctx, cfg->hidden % 256 == 0 && cfg->ffn % 256 == 0, SKN_ERR_SHAPE,
                "skn_llama_create: hidden and ffn must be multiples of 256");
    SKN_REQUIRE(ctx, w->layers && w->tok_embd && w->out_norm && w->out_head, SKN_ERR_ARG,
                "skn_llama_create: missing weights");
    SKN_REQUIRE(ctx, (skn_is_core_quant(w->type_embd) || w->type_embd == SKN_TYPE_F32) && skn_is_quant(w->type_head),
                SKN_ERR_TYPE, "skn_llama_create: unsupported embedding / head type");
    for (int l = 0; l < cfg->n_layer; l++) {
        const skn_llama_layer& L = w->layers[l];
        SKN_REQUIRE(ctx, L.wq && L.wk && L.wv && L.wo && L.w_gate && L.w_up && L.w_down && L.attn_norm && L.ffn_norm,
                    SKN_ERR_ARG, "skn_llama_create: layer %d has a null weight", l);
        SKN_REQUIRE(ctx,
                    skn_is_quant(L.type_q) && skn_is_quant(L.type_k) && skn_is_quant(L.type_v) && skn_is_quant(L.type_o) &&
                        skn_is_quant(L.type_gate) && skn_is_quant(L.type_up) && skn_is_quant(L.type_down),
                    SKN_ERR_TYPE, "skn_llama_create: layer %d has an unsupported weight type", l);
        // (the fused kernels and the GEMMs read 16-byte vectors from these)
        const uintptr_t all = (uintptr_t)L.wq | (uintptr_t)L.wk | (uintptr_t)L.wv | (uintptr_t)L.wo | (uintptr_t)L.w_gate |
                              (uintptr_t)L.w_up | (uintptr_t)L.w_down | (uintptr_t)L.attn_norm | (uintptr_t)L.ffn_norm;
        SKN_REQUIRE(ctx, (all & 15) == 0, SKN_ERR_ARG, "skn_llama_create: the weights of layer %d must be 16-byte aligned", l);
    }
    skn_llama* m = new (std::nothrow) skn_llama();
    SKN_REQUIRE(ctx, m != nullptr, SKN_ERR_OOM, "skn_llama_create: host allocation failed");
    m->cfg = *cfg;
    if (m->cfg.n_kv_head == 0) m->cfg.n_kv_head = cfg->n_head;
    m->w = *w;
    m->layers.assign(w->layers, w->layers + cfg->n_layer);
    m->w.layers = m->layers.data();
    int rc = SKN_OK;
    for (int l = 0; l < cfg->n_layer && rc == SKN_OK; l++) {
        skn_kv* kv = nullptr;
        rc = skn_kv_create(ctx, 1, m->cfg.n_kv_head, cfg->head_dim, cfg->page_tokens, cfg->max_tokens, &kv);
        if (rc == SKN_OK) m->kv.push_back(kv);
    }
    const size_t H = cfg->hidden, F = cfg->ffn;
    const int max_splits = (cfg->max_tokens + 63) / 64;
    auto A = [&](auto** p, size_t n) {
        if (rc == SKN_OK) rc = dev_alloc(ctx, m, p, n);
    };
    A(&m->x, H); A(&m->xn, H); A(&m->q, 3 * H); A(&m->att, H); A(&m->proj, H);
    if (rc == SKN_OK) {  // q, k, v are one buffer so that the three projections can be one launch
        m->k = m->q + H;
        m->v = m->k + (size_t)m->cfg.n_kv_head * cfg->head_dim;
    }
    A(&m->gate, F); A(&m->up, F); A(&m->mid, F); A(&m->logits, (size_t)cfg->vocab);
    A(&m->attn_partial, (size_t)cfg->n_head * max_splits * (cfg->head_dim + 2));
    A(&m->attn_counters, (size_t)cfg->n_head);
    if (rc == SKN_OK && hipMemsetAsync(m->attn_counters, 0, (size_t)cfg->n_head * sizeof(int), ctx->stream) != hipSuccess) {
        (void)hipGetLastError();
        rc = skn_fail(ctx, SKN_ERR_HIP, "skn_llama_create: clearing the attention counters failed");
    }
    A(&m->state, (size_t)4);
    A(&m->inv_freq, (size_t)cfg->head_dim / 2);
    if (rc == SKN_OK) {
        std::vector<double> f(cfg->head_dim / 2);
        for (int i = 0; i < cfg->head_dim / 2; i++) f[i] = pow((double)cfg->rope_base, -2.0 * i / cfg->head_dim);
        if (hipMemcpy(m->inv_freq, f.data(), f.size() * sizeof(double), hipMemcpyHostToDevice) != hipSuccess) {
            (void)hipGetLastError();
            rc = skn_fail(ctx, SKN_ERR_HIP, "skn_llama_create: uploading the rotary frequencies failed");
        }
    }
    m->tokens_cap = cfg->max_tokens;
    A(&m->tokens_out, (size_t)m->tokens_cap);
    if (rc != SKN_OK) {
        skn_llama_free(ctx, m);
        return rc;
    }
    *out = m;
    return SKN_OK;
}

int skn_llama_free(skn_ctx* ctx, skn_llama* m) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_llama_free: ctx is null");
    if (!m) return SKN_OK;
    (void)hipStreamSynchronize(ctx->stream);
    drop_graph(m);
    for (skn_kv* kv : m->kv) skn_kv_free(ctx, kv);
    for (void* p : m->owned) (void)hipFree(p);
    ctx->stat_expanded_bytes -= m->expanded_bytes;
    delete m;
    return SKN_OK;
}

int skn_llama_reset(skn_ctx* ctx, skn_llama* m) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_llama_reset: ctx is null");
    SKN_REQUIRE(ctx, m != nullptr, SKN_ERR_ARG, "skn_llama_reset: model is null");
    for (skn_kv* kv : m->kv) SKN_TRY(skn_kv_reset(ctx, kv, 0));
    m->pos = 0;
    return SKN_OK;
}

// the expanded copy of matrix `which` of layer l, made on first use
static int expanded_copy(skn_ctx* ctx, skn_llama* m, int l, int which, int type, const void* w, int n, int k, const void** out) {
    if (m->expanded.empty()) m->expanded.assign((size_t)m->cfg.n_layer * 7, nullptr);
    void*& slot = m->expanded[(size_t)l * 7 + which];
    if (!slot) {
        uint8_t* p = nullptr;
        SKN_TRY(dev_alloc(ctx, m, &p, skn_gemm_expanded_size(n, k)));
        const int rc = skn_gemm_expand(ctx, type, w, n, k, p);
        if (rc != SKN_OK) {
            dev_release(m, &p);
            return rc;
        }
        slot = p;
        m->expanded_bytes += (long long)skn_gemm_expanded_size(n, k);
        ctx->stat_expanded_bytes += (long long)skn_gemm_expanded_size(n, k);
    }
    *out = slot;
    return SKN_OK;
}

// Prompt rows times up to three matrices of any formats, one activation source (fp32 rows, with RMSNorm when norm_w
// is given).  Q4_K and Q6_K matrices go behind the fused activation pass of their GEMMs -- the row-wise work inside
// the pass, one pass per format, a residual (`accumulate`) in the store --, the others through a norm, a bf16
// conversion, skn_gemm_q per matrix and an add.
int project_rows(skn_ctx* ctx, skn_llama* m, const int* types, const void* const* blocks, const int* rows, float* const* outs,
                 int count, int k, const float* x, const float* norm_w, int T, int accumulate) {
    const skn_llama_config& c = m->cfg;
    const skn_gemm_src src = {norm_w ? SKN_SRC_RMSNORM : SKN_SRC_F32, x, norm_w, norm_w ? c.rms_eps : 0.f};
    skn_gemm_seg q4[3], q6[3];
    int n4 = 0, n6 = 0;
    bool plain = false;
    for (int i = 0; i < count; i++) {
        if (types[i] == SKN_TYPE_Q4_K && k <= 16384) q4[n4++] = {blocks[i], rows[i], outs[i], accumulate};
        else if (types[i] == SKN_TYPE_Q6_K && skn_gemm_q6k_direct_ok(ctx, rows[i], k, T)) q6[n6++] = {blocks[i], rows[i], outs[i], accumulate};
        else plain = true;
    }
    if (n4) SKN_TRY(skn_gemm_q4k_multi(ctx, q4, n4, k, src, T));
    if (n6) SKN_TRY(skn_gemm_q6k_multi(ctx, q6, n6, k, src, T));
    if (!plain) return SKN_OK;
    if (norm_w) {
        skn_launch(ctx, rmsnorm_rows_kernel, dim3(T), dim3(256), 0, x, norm_w, m->pxn, k, c.rms_eps);
        SKN_LAUNCH_CHECK(ctx);
    }
    SKN_TRY(to_bf16(ctx, norm_w ? m->pxn : x, m->pb16, (int64_t)T * k));
    for (int i = 0; i < count; i++) {
        const bool fused = (types[i] == SKN_TYPE_Q4_K && k <= 16384) || (types[i] == SKN_TYPE_Q6_K && skn_gemm_q6k_direct_ok(ctx, rows[i], k, T));
        if (fused) continue;
        if (accumulate) {
            SKN_TRY(skn_gemm_q(ctx, types[i], blocks[i], rows[i], k, m->pb16, T, m->pproj));
            skn_launch(ctx, add_rows_kernel, dim3(nblk((int64_t)T * rows[i])), dim3(256), 0, outs[i], (const float*)m->pproj,
                       (int64_t)T * rows[i]);
            SKN_LAUNCH_CHECK(ctx);
        } else {
            SKN_TRY(skn_gemm_q(ctx, types[i], blocks[i], rows[i], k, m->pb16, T, outs[i]));
        }
    }
    return SKN_OK;
}

int skn_llama_prefill(skn_ctx* ctx, skn_llama* m, const int32_t* tokens_host, int n_tokens, int32_t* next_token_host) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_llama_prefill: ctx is null");
    SKN_REQUIRE(ctx, m && tokens_host, SKN_ERR_ARG, "skn_llama_prefill: null pointer");
    SKN_REQUIRE(ctx, n_tokens > 0, SKN_ERR_ARG, "skn_llama_prefill: the prompt is empty");
    const skn_llama_config& c = m->cfg;
    SKN_REQUIRE(ctx, m->pos + n_tokens <= c.max_tokens, SKN_ERR_POOL, "sequence is full (%d tokens, capacity %d)",
                m->pos + n_tokens, c.max_tokens);
    for (int i = 0; i < n_tokens; i++)
        SKN_REQUIRE(ctx, tokens_host[i] >= 0 && tokens_host[i] < c.vocab, SKN_ERR_RANGE,
                    "skn_llama_prefill: token %d of a vocabulary of %d", tokens_host[i], c.vocab);
    const int T = n_tokens, H = c.hidden, F = c.ffn, NH = c.n_head, D = c.head_dim, pos0 = m->pos;
    const int KVH = c.n_kv_head, KVD = KVH * D;
    SKN_TRY(ensure_prompt_buffers(ctx, m, T));
    SKN_HIP(ctx, hipMemcpyAsync(m->ptok, tokens_host, (size_t)T * sizeof(int32_t), hipMemcpyHostToDevice, ctx->stream));
    SKN_HIP(ctx, hipStreamSynchronize(ctx->stream));
    skn_launch(ctx, set_state_kernel, dim3(1), dim3(64), 0, m->state, 0, pos0);
    SKN_LAUNCH_CHECK(ctx);
    skn_launch(ctx, iota_kernel, dim3(nblk(T)), dim3(256), 0, m->pnctx, T, pos0 + 1);
    SKN_LAUNCH_CHECK(ctx);
    skn_launch(ctx, embed_rows_kernel, dim3(T), dim3(256), 0, (const uint8_t*)m->w.tok_embd, m->w.type_embd, H,
               (const int32_t*)m->ptok, m->px);
    SKN_LAUNCH_CHECK(ctx);
    const float scale = 1.0f / sqrtf((float)D);
    int n_splits = skn_attn_splits(ctx, T * NH, pos0 + T);
    // (the option attn.splits may ask for more than the partials buffer of ensure_prompt_buffers holds)
    n_splits = std::min(n_splits, 1 + 4 * ctx->compute_units / (T * NH));
    for (int l = 0; l < c.n_layer; l++) {
        const skn_llama_layer& L = m->layers[l];
        skn_kv* kv = m->kv[l];
        // Q4_K weights: the GEMM's preparation pass takes the fp32 rows and does the row-wise work before them
        const bool q4k_qkv = H <= 16384 && L.type_q == SKN_TYPE_Q4_K && L.type_k == SKN_TYPE_Q4_K && L.type_v == SKN_TYPE_Q4_K;
        const bool q4k_o = H <= 16384 && L.type_o == SKN_TYPE_Q4_K;
        const bool q4k_gu = H <= 16384 && L.type_gate == SKN_TYPE_Q4_K && L.type_up == SKN_TYPE_Q4_K;
        const bool q4k_down = F <= 16384 && L.type_down == SKN_TYPE_Q4_K;
        SKN_TRY(skn_kv_reserve(ctx, kv, 0, pos0 + T));
        // other formats with the option llama.expand_weights: their fp16-pair copies are kept, and the general GEMM
        // takes the fp32 rows as the Q4_K one does (norm and rounding inside its activation pass, residual in its store)
        const bool expand = ctx->opt_llama_expand != 0 && H % 64 == 0 && F % 64 == 0;
        if (q4k_qkv) {  // RMSNorm inside the activation pass, one launch for the three projections
            const skn_gemm_seg qkv[3] = {{L.wq, H, m->pq, 0}, {L.wk, KVD, m->pk, 0}, {L.wv, KVD, m->pv, 0}};
            const skn_gemm_src src = {SKN_SRC_RMSNORM, m->px, L.attn_norm, c.rms_eps};
            SKN_TRY(skn_gemm_q4k_multi(ctx, qkv, 3, H, src, T));
        } else if (expand) {  // Q4_K matrices of the group on their own kernel, the others through their kept copies
            const int types[3] = {L.type_q, L.type_k, L.type_v}, rows[3] = {H, KVD, KVD};
            const void* blocks[3] = {L.wq, L.wk, L.wv};
            float* outs[3] = {m->pq, m->pk, m->pv};
            skn_gemm_seg q4[3], ex[3];
            int n4 = 0, nx = 0;
            for (int i = 0; i < 3; i++) {
                if (types[i] == SKN_TYPE_Q4_K && H <= 16384) {
                    q4[n4++] = {blocks[i], rows[i], outs[i], 0};
                } else {
                    ex[nx] = {nullptr, rows[i], outs[i], 0};
                    SKN_TRY(expanded_copy(ctx, m, l, i, types[i], blocks[i], rows[i], H, &ex[nx].w));
                    nx++;
                }
            }
            const skn_gemm_src src = {SKN_SRC_RMSNORM, m->px, L.attn_norm, c.rms_eps};
            if (n4) SKN_TRY(skn_gemm_q4k_multi(ctx, q4, n4, H, src, T));
            if (nx) SKN_TRY(skn_gemm_expanded_multi(ctx, ex, nx, H, src, T));
        } else {
            const int types[3] = {L.type_q, L.type_k, L.type_v}, rows[3] = {H, KVD, KVD};
            const void* blocks[3] = {L.wq, L.wk, L.wv};
            float* outs[3] = {m->pq, m->pk, m->pv};
            SKN_TRY(project_rows(ctx, m, types, blocks, rows, outs, 3, H, m->px, L.attn_norm, T, 0));
        }
        skn_launch(ctx, rope_store_kernel, dim3(T, NH), dim3(D / 2), 0, m->pq, (const float*)m->pk, (const float*)m->pv,
                   kv->k_pool, kv->v_pool, (const int32_t*)kv->page_table_dev, (const int32_t*)(m->state + 1), NH, KVH, D,
                   kv->page_tokens, log2((double)c.rope_base));
        SKN_LAUNCH_CHECK(ctx);
        // query row t attends to the first pos0 + t + 1 tokens of the (single) sequence
        if (D <= 128)
            SKN_TRY(skn_attn_prefill_launch(ctx, kv, 0, m->pq, T, pos0 + 1, scale, m->patt, NH));
        else
            SKN_TRY(skn_attn_launch_ex(ctx, kv, m->pq, m->pnctx, T, 0, n_splits, m->ppartial, m->pcounters, scale, m->patt, NH));
        if (q4k_o) {  // the residual is added by the GEMM's store
            const skn_gemm_seg wo = {L.wo, H, m->px, 1};
            const skn_gemm_src src = {SKN_SRC_F32, m->patt, nullptr, 0.f};
            SKN_TRY(skn_gemm_q4k_multi(ctx, &wo, 1, H, src, T));
        } else if (expand) {
            skn_gemm_seg wo = {nullptr, H, m->px, 1};
            SKN_TRY(expanded_copy(ctx, m, l, 3, L.type_o, L.wo, H, H, &wo.w));
            const skn_gemm_src src = {SKN_SRC_F32, m->patt, nullptr, 0.f};
            SKN_TRY(skn_gemm_expanded_multi(ctx, &wo, 1, H, src, T));
        } else {
            const void* blocks[1] = {L.wo};
            float* outs[1] = {m->px};
            SKN_TRY(project_rows(ctx, m, &L.type_o, blocks, &H, outs, 1, H, m->patt, nullptr, T, 1));
        }
        if (q4k_gu) {  // RMSNorm inside the activation pass, SwiGLU inside the store: gate and up never reach memory
            const skn_gemm_seg gu[2] = {{L.w_gate, F, m->pmid, 0}, {L.w_up, F, m->pmid, 0}};
            const skn_gemm_src src = {SKN_SRC_RMSNORM, m->px, L.ffn_norm, c.rms_eps};
            SKN_TRY(skn_gemm_q4k_multi(ctx, gu, 2, H, src, T, true));
        } else if (expand) {
            const int types[2] = {L.type_gate, L.type_up};
            const void* blocks[2] = {L.w_gate, L.w_up};
            float* outs[2] = {m->pgate, m->pup};
            const skn_gemm_src src = {SKN_SRC_RMSNORM, m->px, L.ffn_norm, c.rms_eps};
            for (int i = 0; i < 2; i++) {
                skn_gemm_seg seg = {blocks[i], F, outs[i], 0};
                if (types[i] == SKN_TYPE_Q4_K && H <= 16384) {
                    SKN_TRY(skn_gemm_q4k_multi(ctx, &seg, 1, H, src, T));
                } else {
                    SKN_TRY(expanded_copy(ctx, m, l, 4 + i, types[i], blocks[i], F, H, &seg.w));
                    SKN_TRY(skn_gemm_expanded_multi(ctx, &seg, 1, H, src, T));
                }
            }
            skn_launch(ctx, swiglu_rows_kernel, dim3(nblk((int64_t)T * F)), dim3(256), 0, (const float*)m->pgate,
                       (const float*)m->pup, m->pmid, (int64_t)T * F);
            SKN_LAUNCH_CHECK(ctx);
        } else {
            const int types[2] = {L.type_gate, L.type_up}, rows[2] = {F, F};
            const void* blocks[2] = {L.w_gate, L.w_up};
            float* outs[2] = {m->pgate, m->pup};
            SKN_TRY(project_rows(ctx, m, types, blocks, rows, outs, 2, H, m->px, L.ffn_norm, T, 0));
            skn_launch(ctx, swiglu_rows_kernel, dim3(nblk((int64_t)T * F)), dim3(256), 0, (const float*)m->pgate,
                       (const float*)m->pup, m->pmid, (int64_t)T * F);
            SKN_LAUNCH_CHECK(ctx);
        }
        if (q4k_down) {
            const skn_gemm_seg down = {L.w_down, H, m->px, 1};  // residual added by the store
            const skn_gemm_src mid = {SKN_SRC_F32, m->pmid, nullptr, 0.f};
            SKN_TRY(skn_gemm_q4k_multi(ctx, &down, 1, F, mid, T));
        } else if (expand) {
            skn_gemm_seg down = {nullptr, H, m->px, 1};
            SKN_TRY(expanded_copy(ctx, m, l, 6, L.type_down, L.w_down, H, F, &down.w));
            const skn_gemm_src mid = {SKN_SRC_F32, m->pmid, nullptr, 0.f};
            SKN_TRY(skn_gemm_expanded_multi(ctx, &down, 1, F, mid, T));
        } else {
            const void* blocks[1] = {L.w_down};
            float* outs[1] = {m->px};
            SKN_TRY(project_rows(ctx, m, &L.type_down, blocks, &H, outs, 1, F, m->pmid, nullptr, T, 1));
        }
        // the cache of this layer now holds pos0 + T tokens
        kv->len[0] = pos0 + T;
    }
    // logits of the last prompt token only
    skn_launch(ctx, rmsnorm_rows_kernel, dim3(1), dim3(256), 0, (const float*)(m->px + (size_t)(T - 1) * H),
               m->w.out_norm, m->xn, H, c.rms_eps);
    SKN_LAUNCH_CHECK(ctx);
    SKN_TRY(skn_matvec_q(ctx, m->w.type_head, m->w.out_head, c.vocab, H, m->xn, m->logits));
    skn_launch(ctx, finish_step_kernel, dim3(1), dim3(1024), 0, (const float*)m->logits, c.vocab, m->state,
               m->tokens_out, 0);
    SKN_LAUNCH_CHECK(ctx);
    m->pos = pos0 + T;
    int32_t next = 0;
    SKN_HIP(ctx, hipMemcpyAsync(&next, m->tokens_out, sizeof(int32_t), hipMemcpyDeviceToHost, ctx->stream));
    SKN_HIP(ctx, hipStreamSynchronize(ctx->stream));
    if (next_token_host) *next_token_host = next;
    return SKN_OK;
}

int skn_llama_decode(skn_ctx* ctx, skn_llama* m, int32_t first_token, int n_steps, int32_t* tokens_out_host) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_llama_decode: ctx is null");
    SKN_REQUIRE(ctx, m != nullptr, SKN_ERR_ARG, "skn_llama_decode: model is null");
    SKN_REQUIRE(ctx, n_steps >= 0, SKN_ERR_ARG, "skn_llama_decode: negative step count");
    if (n_steps == 0) return SKN_OK;
    const skn_llama_config& c = m->cfg;
    SKN_REQUIRE(ctx, tokens_out_host != nullptr, SKN_ERR_ARG, "skn_llama_decode: tokens_out is null");
    SKN_REQUIRE(ctx, first_token >= 0 && first_token < c.vocab, SKN_ERR_RANGE,
                "skn_llama_decode: token %d of a vocabulary of %d", first_token, c.vocab);
    SKN_REQUIRE(ctx, m->pos + n_steps <= c.max_tokens, SKN_ERR_POOL, "sequence is full (%d tokens, capacity %d)",
                m->pos + n_steps, c.max_tokens);
    SKN_REQUIRE(ctx, !ctx->prof_on, SKN_ERR_STATE, "skn_llama_decode: not available while per-launch timing is on");
    // every page the run will touch is mapped now; the step itself never talks to the host
    for (skn_kv* kv : m->kv) SKN_TRY(skn_kv_reserve(ctx, kv, 0, m->pos + n_steps));
    skn_launch(ctx, set_state_kernel, dim3(1), dim3(64), 0, m->state, (int)first_token, m->pos);
    SKN_LAUNCH_CHECK(ctx);
    // A split count for the longest context of this run, rounded up to a power of two of 128-token units (the kernel
    // derives its ranges from the actual length, so one captured step serves every position up to there): the step is
    // captured again only when a sequence grows past 128, 256, 512, ... tokens, and a short context is not cut into
    // more pieces than it has work for (sixteen splits of 600 tokens cost 2 % of the step against eight).
    int n_splits = 1;
    while (n_splits * 128 < m->pos + n_steps) n_splits *= 2;
    n_splits = std::min(n_splits, skn_attn_splits(ctx, c.n_head, c.max_tokens));
    if (ctx->opt_llama_graph == 0) {
        for (int i = 0; i < n_steps; i++) SKN_TRY(decode_step(ctx, m, n_splits));
    } else {
        // a captured step has the kernel set of the options (and the stream) it was captured with baked in
        if (m->graph_exec && (m->graph_splits != n_splits || m->graph_generation != ctx->opt_generation)) drop_graph(m);
        if (!m->graph_exec) {
            SKN_HIP(ctx, hipStreamSynchronize(ctx->stream));
            SKN_HIP(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
            int rc = decode_step(ctx, m, n_splits);
            hipGraph_t g = nullptr;
            hipError_t e = hipStreamEndCapture(ctx->stream, &g);
            if (rc != SKN_OK) {
                if (g) (void)hipGraphDestroy(g);
                return rc;
            }
            if (e != hipSuccess) return skn_fail(ctx, SKN_ERR_HIP, "stream capture failed: %s", hipGetErrorString(e));
            m->graph = g;
            SKN_HIP(ctx, hipGraphInstantiate(&m->graph_exec, m->graph, nullptr, nullptr, 0));
            m->graph_splits = n_splits;
            m->graph_generation = ctx->opt_generation;
            ctx->stat_captures++;
        }
        for (int i = 0; i < n_steps; i++) SKN_HIP(ctx, hipGraphLaunch(m->graph_exec, ctx->stream));
    }
    SKN_HIP(ctx, hipMemcpyAsync(tokens_out_host, m->tokens_out, (size_t)n_steps * sizeof(int32_t), hipMemcpyDeviceToHost,
                                ctx->stream));
    SKN_HIP(ctx, hipStreamSynchronize(ctx->stream));
    m->pos += n_steps;
    for (skn_kv* kv : m->kv) kv->len[0] = m->pos;
    return SKN_OK;
}

int skn_llama_logits(skn_ctx* ctx, skn_llama* m, const float** logits_dev) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_llama_logits: ctx is null");
    SKN_REQUIRE(ctx, m && logits_dev, SKN_ERR_ARG, "skn_llama_logits: null pointer");
    *logits_dev = m->logits;
    return SKN_OK;
}

}  // extern "C"
