// Paged KV cache object shared by the cache kernels, decode attention and the decoder.
#pragma once
#include "common.h"

struct skn_kv {
    int n_seq = 0, n_head = 0, head_dim = 0, page_tokens = 0, max_tokens = 0;
    int pages_per_seq = 0, n_pages = 0;
    // page p, head h, slot s, element e lives at ((p * n_head + h) * page_tokens + s) * head_dim + e:
    // one head's tokens of a page are contiguous, so attention streams page_tokens * head_dim * 2 bytes runs.
    uint16_t* k_pool = nullptr;
    uint16_t* v_pool = nullptr;
    int32_t* page_table_dev = nullptr;  // [n_seq][pages_per_seq], -1 = not mapped
    int32_t* len_dev = nullptr;         // [n_seq] tokens held, the kernels' source of append positions
    int32_t* nctx_dev = nullptr;        // [n_seq] staging for explicit attention lengths
    int* ticket_dev = nullptr;          // workgroups of an append launch count themselves in (zero between launches)
    std::vector<int32_t> page_table;    // host mirror
    std::vector<int32_t> len;           // host mirror
    std::vector<int32_t> free_pages;    // stack of unmapped page ids
    std::vector<int32_t> nctx_host;     // keeps explicit attention lengths alive while their upload is queued
};

// Maps pages so that sequence `seq` can hold `new_len` tokens; uploads new table entries on the stream.
int skn_kv_reserve(skn_ctx* ctx, skn_kv* kv, int seq, int new_len);

// Counts n more tokens into a sequence whose rows were written by a kernel outside the cache code (pages reserved
// by the caller): host mirror and device length.
int skn_kv_advance_len(skn_ctx* ctx, skn_kv* kv, int seq, int n);

// Attention over `kv` with per-sequence lengths taken from a device array; max_ctx bounds them (host knowledge).
int skn_attn_launch(skn_ctx* ctx, skn_kv* kv, const float* q_dev, const int32_t* nctx_dev, int max_ctx, float scale,
                    float* out_dev);
int skn_attn_launch_ex(skn_ctx* ctx, skn_kv* kv, const float* q_dev, const int32_t* nctx_dev, int n_queries,
                       int seq_fixed, int n_splits, float* partial, int* counters, float scale, float* out_dev,
                       int n_q_head = 0);  // query heads (a multiple of the cached heads; 0: as many)
int skn_attn_splits(skn_ctx* ctx, int pairs, int max_ctx);
// Causal attention of n_queries rows of one sequence: row t attends to its first first_ctx + t tokens (head_dim 64 / 128).
int skn_attn_prefill_launch(skn_ctx* ctx, skn_kv* kv, int seq, const float* q_dev, int n_queries, int first_ctx, float scale,
                            float* out_dev, int n_q_head = 0);
