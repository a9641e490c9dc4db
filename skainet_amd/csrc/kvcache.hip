// Device-resident paged KV cache: create / reset / append / gather.  Pure fp16 data movement (bit-exact).
//
// Layout: two pools (K and V) of n_pages pages; a page holds page_tokens tokens of every head, head-major
// ([head][slot][head_dim]), so the rows of one head are contiguous inside a page.  A per-sequence page table
// maps token t to page table[seq][t / page_tokens], slot t % page_tokens.  Pages are handed out on demand by
// the host from a free stack; token counts live on the device (the append kernels read their positions
// there, which keeps a captured decode step replayable) and are mirrored on the host for argument checks.
#include "kv.h"

namespace {

constexpr int kMaxAppend = 64;  // entries per launch of the scattered append

struct AppendArgs {
    int32_t seq[kMaxAppend];
    int32_t rank[kMaxAppend];  // number of earlier entries of this launch with the same sequence
};

// grid (n_entries, n_head); one 16-byte chunk per thread, head_dim / 8 chunks per row.
__global__ void kv_append_kernel(uint16_t* __restrict__ k_pool, uint16_t* __restrict__ v_pool,
                                 const int32_t* __restrict__ table, int32_t* len, int* ticket,
                                 const uint16_t* __restrict__ k_in, const uint16_t* __restrict__ v_in, AppendArgs a,
                                 int n_head, int head_dim, int page_tokens, int pages_per_seq) {
    const int i = blockIdx.x, h = blockIdx.y;
    const int seq = a.seq[i];
    const int t = len[seq] + a.rank[i];
    const int page = table[seq * pages_per_seq + t / page_tokens];
    const int slot = t % page_tokens;
    const size_t dst = (((size_t)page * n_head + h) * page_tokens + slot) * head_dim;
    const size_t src = ((size_t)i * n_head + h) * head_dim;
    const int chunks = head_dim >> 3;
    for (int c = threadIdx.x; c < chunks; c += blockDim.x) {
        reinterpret_cast<uint4*>(k_pool + dst)[c] = reinterpret_cast<const uint4*>(k_in + src)[c];
        reinterpret_cast<uint4*>(v_pool + dst)[c] = reinterpret_cast<const uint4*>(v_in + src)[c];
    }
    // The lengths advance once every workgroup of the launch has read them: each takes a ticket after its read (the
    // read's value has been used above, so it has completed), and the holder of the last ticket counts the new tokens
    // in and returns the ticket counter to zero for the next launch.
    if (threadIdx.x == 0) {
        const int total = gridDim.x * gridDim.y;
        // (Relaxed, at device scope.  What orders the other workgroups' reads of len before the last holder's update is
        // the hardware: a workgroup's read has returned -- its value addressed the stores above -- before its thread 0
        // issues the ticket.  In the language's memory model that is a race; the acquire-release form, which removes it,
        // makes every workgroup write its L2 back before the ticket and was measured at 8.5 - 9.3 us per step against
        // 6.1 - 6.2 us, so it is not used.)
        if (__hip_atomic_fetch_add(ticket, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == total - 1) {
            for (int e = 0; e < (int)gridDim.x; e++) len[a.seq[e]] += 1;
            __hip_atomic_store(ticket, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// grid (n_tokens, n_head): consecutive tokens of one sequence starting at t0 (append) or copied out (gather).
template <bool GATHER>
__global__ void kv_run_kernel(uint16_t* __restrict__ k_pool, uint16_t* __restrict__ v_pool,
                              const int32_t* __restrict__ table, uint16_t* __restrict__ k_lin,
                              uint16_t* __restrict__ v_lin, int seq, int t0, int n_head, int head_dim, int page_tokens,
                              int pages_per_seq) {
    const int i = blockIdx.x, h = blockIdx.y;
    const int t = t0 + i;
    const int page = table[seq * pages_per_seq + t / page_tokens];
    const int slot = t % page_tokens;
    const size_t paged = (((size_t)page * n_head + h) * page_tokens + slot) * head_dim;
    const size_t lin = ((size_t)i * n_head + h) * head_dim;
    const int chunks = head_dim >> 3;
    for (int c = threadIdx.x; c < chunks; c += blockDim.x) {
        if (GATHER) {
            reinterpret_cast<uint4*>(k_lin + lin)[c] = reinterpret_cast<const uint4*>(k_pool + paged)[c];
            reinterpret_cast<uint4*>(v_lin + lin)[c] = reinterpret_cast<const uint4*>(v_pool + paged)[c];
        } else {
            reinterpret_cast<uint4*>(k_pool + paged)[c] = reinterpret_cast<const uint4*>(k_lin + lin)[c];
            reinterpret_cast<uint4*>(v_pool + paged)[c] = reinterpret_cast<const uint4*>(v_lin + lin)[c];
        }
    }
}

__global__ void kv_set_len_kernel(int32_t* len, int seq, int n_seq, int value, int delta) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n_seq && (seq < 0 || i == seq)) len[i] = delta ? len[i] + value : value;
}

void release_pages(skn_kv* kv, int seq) {
    for (int p = 0; p < kv->pages_per_seq; p++) {
        int32_t& e = kv->page_table[(size_t)seq * kv->pages_per_seq + p];
        if (e >= 0) {
            kv->free_pages.push_back(e);
            e = -1;
        }
    }
    kv->len[seq] = 0;
}

}  // namespace

int skn_kv_reserve(skn_ctx* ctx, skn_kv* kv, int seq, int new_len) {
    SKN_REQUIRE(ctx, new_len <= kv->max_tokens, SKN_ERR_POOL, "sequence %d is full (%d tokens, capacity %d)", seq,
                new_len, kv->max_tokens);
    const int need = (new_len + kv->page_tokens - 1) / kv->page_tokens;
    int32_t* row = &kv->page_table[(size_t)seq * kv->pages_per_seq];
    int first_new = -1, last_new = -1;
    for (int p = 0; p < need; p++) {
        if (row[p] >= 0) continue;
        SKN_REQUIRE(ctx, !kv->free_pages.empty(), SKN_ERR_POOL, "KV page pool exhausted (%d pages)", kv->n_pages);
        row[p] = kv->free_pages.back();
        kv->free_pages.pop_back();
        if (first_new < 0) first_new = p;
        last_new = p;
    }
    if (first_new >= 0) {
        // the host vector outlives the copy: the call is synchronous for pageable memory
        SKN_HIP(ctx, hipMemcpyAsync(kv->page_table_dev + (size_t)seq * kv->pages_per_seq + first_new, row + first_new,
                                    (size_t)(last_new - first_new + 1) * sizeof(int32_t), hipMemcpyHostToDevice,
                                    ctx->stream));
    }
    return SKN_OK;
}

int skn_kv_advance_len(skn_ctx* ctx, skn_kv* kv, int seq, int n) {
    skn_launch(ctx, kv_set_len_kernel, dim3((kv->n_seq + 63) / 64), dim3(64), 0, kv->len_dev, seq, kv->n_seq, n, 1);
    SKN_LAUNCH_CHECK(ctx);
    kv->len[seq] += n;
    return SKN_OK;
}

extern "C" {

int skn_kv_create(skn_ctx* ctx, int n_seq, int n_head, int head_dim, int page_tokens, int max_tokens, skn_kv** out) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_kv_create: ctx is null");
    SKN_REQUIRE(ctx, out != nullptr, SKN_ERR_ARG, "skn_kv_create: out is null");
    *out = nullptr;
    SKN_REQUIRE(ctx, n_seq > 0 && n_head > 0 && head_dim > 0 && page_tokens > 0 && max_tokens > 0, SKN_ERR_ARG,
                "skn_kv_create: sizes must be positive");
    SKN_REQUIRE(ctx, head_dim % 8 == 0, SKN_ERR_SHAPE, "skn_kv_create: head_dim (%d) must be a multiple of 8", head_dim);
    skn_kv* kv = new (std::nothrow) skn_kv();
    SKN_REQUIRE(ctx, kv != nullptr, SKN_ERR_OOM, "skn_kv_create: host allocation failed");
    kv->n_seq = n_seq;
    kv->n_head = n_head;
    kv->head_dim = head_dim;
    kv->page_tokens = page_tokens;
    kv->max_tokens = max_tokens;
    kv->pages_per_seq = (max_tokens + page_tokens - 1) / page_tokens;
    kv->n_pages = n_seq * kv->pages_per_seq;
    const size_t page_elems = (size_t)n_head * page_tokens * head_dim;
    const size_t pool_bytes = (size_t)kv->n_pages * page_elems * sizeof(uint16_t);
    const size_t table_bytes = (size_t)n_seq * kv->pages_per_seq * sizeof(int32_t);
    hipError_t e = hipMalloc((void**)&kv->k_pool, pool_bytes);
    if (e == hipSuccess) e = hipMalloc((void**)&kv->v_pool, pool_bytes);
    if (e == hipSuccess) e = hipMalloc((void**)&kv->page_table_dev, table_bytes);
    if (e == hipSuccess) e = hipMalloc((void**)&kv->len_dev, (size_t)n_seq * sizeof(int32_t));
    if (e == hipSuccess) e = hipMalloc((void**)&kv->nctx_dev, (size_t)n_seq * sizeof(int32_t));
    if (e == hipSuccess) e = hipMalloc((void**)&kv->ticket_dev, 16);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        int rc = skn_fail(ctx, SKN_ERR_OOM, "skn_kv_create: %zu-byte pools: %s", pool_bytes, hipGetErrorString(e));
        skn_kv_free(ctx, kv);
        return rc;
    }
    kv->page_table.assign((size_t)n_seq * kv->pages_per_seq, -1);
    kv->len.assign(n_seq, 0);
    kv->free_pages.reserve(kv->n_pages);
    for (int p = kv->n_pages - 1; p >= 0; p--) kv->free_pages.push_back(p);
    int rc = skn_memset(ctx, kv->page_table_dev, 0xFF, table_bytes);
    if (rc == SKN_OK) rc = skn_memset(ctx, kv->len_dev, 0, (size_t)n_seq * sizeof(int32_t));
    if (rc == SKN_OK) rc = skn_memset(ctx, kv->nctx_dev, 0, (size_t)n_seq * sizeof(int32_t));
    if (rc == SKN_OK) rc = skn_memset(ctx, kv->ticket_dev, 0, 16);
    if (rc != SKN_OK) {
        skn_kv_free(ctx, kv);
        return rc;
    }
    *out = kv;
    return SKN_OK;
}

int skn_kv_free(skn_ctx* ctx, skn_kv* kv) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_kv_free: ctx is null");
    if (!kv) return SKN_OK;
    (void)hipStreamSynchronize(ctx->stream);
    if (kv->k_pool) (void)hipFree(kv->k_pool);
    if (kv->v_pool) (void)hipFree(kv->v_pool);
    if (kv->page_table_dev) (void)hipFree(kv->page_table_dev);
    if (kv->len_dev) (void)hipFree(kv->len_dev);
    if (kv->nctx_dev) (void)hipFree(kv->nctx_dev);
    if (kv->ticket_dev) (void)hipFree(kv->ticket_dev);
    delete kv;
    return SKN_OK;
}

int skn_kv_reset(skn_ctx* ctx, skn_kv* kv, int seq) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_kv_reset: ctx is null");
    SKN_REQUIRE(ctx, kv != nullptr, SKN_ERR_ARG, "skn_kv_reset: kv is null");
    SKN_REQUIRE(ctx, seq >= -1 && seq < kv->n_seq, SKN_ERR_RANGE, "skn_kv_reset: sequence %d of %d", seq, kv->n_seq);
    for (int s = 0; s < kv->n_seq; s++)
        if (seq < 0 || s == seq) release_pages(kv, s);
    // stale table entries are harmless: a page is looked up only below the sequence length
    skn_launch(ctx, kv_set_len_kernel, dim3((kv->n_seq + 63) / 64), dim3(64), 0, kv->len_dev, seq,
                       kv->n_seq, 0, 0);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

int skn_kv_len(skn_ctx* ctx, skn_kv* kv, int seq) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_kv_len: ctx is null");
    SKN_REQUIRE(ctx, kv != nullptr, SKN_ERR_ARG, "skn_kv_len: kv is null");
    SKN_REQUIRE(ctx, seq >= 0 && seq < kv->n_seq, SKN_ERR_RANGE, "skn_kv_len: sequence %d of %d", seq, kv->n_seq);
    return kv->len[seq];
}

int skn_kv_append(skn_ctx* ctx, skn_kv* kv, const uint16_t* k_dev, const uint16_t* v_dev, const int32_t* seq_ids_host,
                  int n) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_kv_append: ctx is null");
    SKN_REQUIRE(ctx, kv != nullptr, SKN_ERR_ARG, "skn_kv_append: kv is null");
    SKN_REQUIRE(ctx, n >= 0, SKN_ERR_ARG, "skn_kv_append: negative count");
    if (n == 0) return SKN_OK;
    SKN_REQUIRE(ctx, k_dev && v_dev && seq_ids_host, SKN_ERR_ARG, "skn_kv_append: null pointer");
    SKN_REQUIRE(ctx, (((uintptr_t)k_dev | (uintptr_t)v_dev) & 15) == 0, SKN_ERR_ARG,
                "skn_kv_append: k/v must be 16-byte aligned");
    // validate the whole list and make sure every target page exists before anything is written
    std::vector<int32_t> extra(kv->n_seq, 0);
    for (int i = 0; i < n; i++) {
        const int s = seq_ids_host[i];
        SKN_REQUIRE(ctx, s >= 0 && s < kv->n_seq, SKN_ERR_RANGE, "skn_kv_append: sequence %d of %d", s, kv->n_seq);
        extra[s]++;
    }
    for (int s = 0; s < kv->n_seq; s++)
        SKN_REQUIRE(ctx, kv->len[s] + extra[s] <= kv->max_tokens, SKN_ERR_POOL,
                    "sequence %d is full (%d tokens, capacity %d)", s, kv->len[s] + extra[s], kv->max_tokens);
    for (int s = 0; s < kv->n_seq; s++)
        if (extra[s]) {
            int rc = skn_kv_reserve(ctx, kv, s, kv->len[s] + extra[s]);
            if (rc != SKN_OK) return rc;
        }
    const size_t row = (size_t)kv->n_head * kv->head_dim;
    std::vector<int32_t> seen(kv->n_seq, 0);
    for (int base = 0; base < n; base += kMaxAppend) {
        const int cnt = n - base < kMaxAppend ? n - base : kMaxAppend;
        AppendArgs a;
        std::fill(seen.begin(), seen.end(), 0);
        for (int i = 0; i < cnt; i++) {
            a.seq[i] = seq_ids_host[base + i];
            a.rank[i] = seen[a.seq[i]]++;
        }
        skn_launch(ctx, kv_append_kernel, dim3(cnt, kv->n_head), dim3(64), 0, kv->k_pool, kv->v_pool, kv->page_table_dev, kv->len_dev, kv->ticket_dev,
                           k_dev + base * row, v_dev + base * row, a, kv->n_head, kv->head_dim, kv->page_tokens, kv->pages_per_seq);
        SKN_LAUNCH_CHECK(ctx);
        for (int i = 0; i < cnt; i++) kv->len[a.seq[i]]++;
    }
    return SKN_OK;
}

int skn_kv_append_run(skn_ctx* ctx, skn_kv* kv, int seq, const uint16_t* k_dev, const uint16_t* v_dev, int n_tokens) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_kv_append_run: ctx is null");
    SKN_REQUIRE(ctx, kv != nullptr, SKN_ERR_ARG, "skn_kv_append_run: kv is null");
    SKN_REQUIRE(ctx, seq >= 0 && seq < kv->n_seq, SKN_ERR_RANGE, "skn_kv_append_run: sequence %d of %d", seq, kv->n_seq);
    SKN_REQUIRE(ctx, n_tokens >= 0, SKN_ERR_ARG, "skn_kv_append_run: negative count");
    if (n_tokens == 0) return SKN_OK;
    SKN_REQUIRE(ctx, k_dev && v_dev, SKN_ERR_ARG, "skn_kv_append_run: null pointer");
    SKN_REQUIRE(ctx, (((uintptr_t)k_dev | (uintptr_t)v_dev) & 15) == 0, SKN_ERR_ARG,
                "skn_kv_append_run: k/v must be 16-byte aligned");
    const int t0 = kv->len[seq];
    int rc = skn_kv_reserve(ctx, kv, seq, t0 + n_tokens);
    if (rc != SKN_OK) return rc;
    skn_launch(ctx, kv_run_kernel<false>, dim3(n_tokens, kv->n_head), dim3(64), 0, kv->k_pool,
                       kv->v_pool, kv->page_table_dev, const_cast<uint16_t*>(k_dev), const_cast<uint16_t*>(v_dev), seq,
                       t0, kv->n_head, kv->head_dim, kv->page_tokens, kv->pages_per_seq);
    SKN_LAUNCH_CHECK(ctx);
    skn_launch(ctx, kv_set_len_kernel, dim3((kv->n_seq + 63) / 64), dim3(64), 0, kv->len_dev, seq,
                       kv->n_seq, n_tokens, 1);
    SKN_LAUNCH_CHECK(ctx);
    kv->len[seq] = t0 + n_tokens;
    return SKN_OK;
}

int skn_kv_gather(skn_ctx* ctx, skn_kv* kv, int seq, int t0, int t1, uint16_t* k_out_dev, uint16_t* v_out_dev) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_kv_gather: ctx is null");
    SKN_REQUIRE(ctx, kv != nullptr, SKN_ERR_ARG, "skn_kv_gather: kv is null");
    SKN_REQUIRE(ctx, seq >= 0 && seq < kv->n_seq, SKN_ERR_RANGE, "skn_kv_gather: sequence %d of %d", seq, kv->n_seq);
    SKN_REQUIRE(ctx, t0 >= 0 && t0 <= t1 && t1 <= kv->len[seq], SKN_ERR_RANGE,
                "skn_kv_gather: tokens [%d, %d) of a sequence holding %d", t0, t1, kv->len[seq]);
    if (t1 == t0) return SKN_OK;
    SKN_REQUIRE(ctx, k_out_dev && v_out_dev, SKN_ERR_ARG, "skn_kv_gather: null pointer");
    SKN_REQUIRE(ctx, (((uintptr_t)k_out_dev | (uintptr_t)v_out_dev) & 15) == 0, SKN_ERR_ARG,
                "skn_kv_gather: outputs must be 16-byte aligned");
    skn_launch(ctx, kv_run_kernel<true>, dim3(t1 - t0, kv->n_head), dim3(64), 0, kv->k_pool, kv->v_pool,
                       kv->page_table_dev, k_out_dev, v_out_dev, seq, t0, kv->n_head, kv->head_dim, kv->page_tokens,
                       kv->pages_per_seq);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

}  // extern "C"
