// Shared internals of libskainet_hip: context, error plumbing, wave-level helpers.  gfx950 only.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <hip/hip_fp16.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/skainet_hip.h"

struct skn_ctx {
    int device = 0;
    hipStream_t stream = nullptr;      // stream in use
    hipStream_t own_stream = nullptr;  // stream created by skn_init
    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
    bool timer_running = false;
    int compute_units = 0;
    size_t lds_per_block = 0;
    std::string err;
    // per-launch kernel timing (skn_prof_start / skn_prof_stop): one start/stop event pair per launch
    bool prof_on = false;
    size_t prof_used = 0;
    std::vector<hipEvent_t> prof_events;
    // tuning options (skn_set_option); 0 = library default
    int opt_q4k_split = 0;  // Q4_K matvec with k split across workgroups (measured alternative): 1 ticket merge, 2 atomic adds
    int opt_q4k_waves = 0, opt_q4k_rows = 0, opt_attn_splits = 0, opt_llama_graph = 1, opt_llama_fused = 1, opt_gemm_tile = 0, opt_matvec_stage = 1, opt_llama_expand = 0, opt_test_rope_table = 0, opt_llama_attn_wide = 1, opt_gemm_q6k_fused = 1;
    int opt_generation = 0;          // bumped by every skn_set_option / skn_set_stream: captured work is stamped with it
    bool profiler_attached = false;  // a rocprofiler tool library is loaded into this process: graphs are not replayed
    long long stat_launches = 0, stat_captures = 0;  // kernel launches issued (or recorded) / decode-step graphs captured
    long long stat_expanded_bytes = 0;               // device bytes held by the decoders' expanded weight copies
    // scratch for split-context attention partials, grown on demand
    void* attn_scratch = nullptr;
    size_t attn_scratch_bytes = 0;
    int* attn_counters = nullptr;  // one per (sequence, head): workgroups of a split attention count themselves in
    int attn_counters_cap = 0;
    // partials and tickets of the split Q4_K matvec (option q4k.split), grown on demand
    void* split_scratch = nullptr;
    size_t split_scratch_bytes = 0;
    int split_scratch_n = 0, split_scratch_slices = 0;
    // prompt attention workspace (K and V of a sequence in matrix-core operand order), grown on demand
    void* prefill_ws = nullptr;
    size_t prefill_ws_bytes = 0;
    // GEMM workspace (fp16 activations, dequantized weight pairs), grown on demand
    void* gemm_ws = nullptr;
    size_t gemm_ws_bytes = 0;
};

// One-time kernel attribute setup (large dynamic LDS), called by skn_init.
int skn_matvec_init(skn_ctx* ctx);
int skn_gemm_init(skn_ctx* ctx);
int skn_attn_init(skn_ctx* ctx);

// Fused Q4_K matvec used by the decoder: up to three [rows_i, k] matrices stacked along the output axis,
// optional RMSNorm of x (norm_w != nullptr) and a store / add-into / SwiGLU epilogue.
struct skn_q4k_segments {
    const uint8_t* w[3];
    int rows[3];
};
// SKN_EPI_ROPE: the three segments are the q, k and v projections of one token.  A wavefront's two rows are
// one rotary pair: q pairs are rotated and stored to y (fp32), k pairs are rotated and stored as fp16 into the
// cache page of the token's position, v pairs are stored as fp16 beside them.
enum { SKN_EPI_STORE = 0, SKN_EPI_ADD = 1, SKN_EPI_SWIGLU = 2, SKN_EPI_ROPE = 3 };
struct skn_kv;
struct skn_rope_epilogue {
    const int32_t* pos_dev = nullptr;     // position of the token (device scalar)
    const int32_t* page_table = nullptr;  // page table row of the token's sequence
    uint16_t* k_pool = nullptr;
    uint16_t* v_pool = nullptr;
    int n_head = 0, head_dim = 0, page_tokens = 0;
    double log2_base = 0.0;  // log2 of the rotary base, in double: the angle pos * base^(-2i/d) is formed in double
    const double* inv_freq = nullptr;  // optional device table base^(-2i/d), i < head_dim / 2 (saves the exp2 per wavefront)
    // SKN_EPI_ADD without a norm (the output projection of an attention block): x is not a finished vector but the
    // unmerged split partials of the decode attention -- x[split][pair][head_dim] unnormalised outputs, merge_ml
    // [split][pair] (max, sum) -- and the staging merges them (skn_attn_launch_unmerged wrote them).  0 splits: plain x.
    const float* merge_ml = nullptr;
    int merge_splits = 0, merge_pairs = 0, merge_head_f4 = 0;  // pairs = query rows x heads, head_f4 = head_dim / 4
};
// Decode attention whose split partials are left unmerged for the consumer above (n_splits >= 2), or merged into out
// (n_splits == 1).  One workgroup of sixteen wavefronts per (split, head, query row); no device counters, no atomics.
// opart: n_splits * n_queries * n_q_head * head_dim floats, ml: two floats per (split, query row, head).
int skn_attn_launch_unmerged(skn_ctx* ctx, skn_kv* kv, const float* q_dev, const int32_t* nctx_dev, int n_queries,
                             int seq_fixed, int n_splits, float* opart, float* ml, float scale, float* out_dev, int n_q_head);
int skn_matvec_q4k_fused(skn_ctx* ctx, const skn_q4k_segments& seg, int n_out, int k, const float* x, const float* norm_w,
                         float eps, float* y, int epi, const skn_rope_epilogue* rope = nullptr, int ggml_type = SKN_TYPE_Q4_K);
// the formats the fused kernels take (every matrix of a launch in the same one; k a multiple of 256)
bool skn_matvec_fusable(int ggml_type);

// Records a failure on the context (or on the context-less slot) and returns `code`.
int skn_fail(skn_ctx* ctx, int code, const char* fmt, ...);

#define SKN_REQUIRE(ctx, cond, code, ...)                         \
    do {                                                          \
        if (!(cond)) return skn_fail((ctx), (code), __VA_ARGS__); \
    } while (0)

#define SKN_HIP(ctx, expr)                                                                             \
    do {                                                                                               \
        hipError_t e_ = (expr);                                                                        \
        if (e_ != hipSuccess)                                                                          \
            return skn_fail((ctx), SKN_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), \
                            __FILE__, __LINE__);                                                       \
    } while (0)

// Call after a kernel launch.
#define SKN_LAUNCH_CHECK(ctx) SKN_HIP((ctx), hipGetLastError())

// Every kernel launch of the library goes through here.  While per-launch timing is on, the launch carries
// its own start/stop events, which read the dispatch's begin and end timestamps (the kernel's duration as a
// profiler reports it, without launch gaps).
template <typename F, typename... Args>
inline void skn_launch(skn_ctx* ctx, F kernel, dim3 grid, dim3 block, size_t lds, Args... args) {
    ctx->stat_launches++;
    if (ctx->prof_on && 2 * ctx->prof_used + 1 < ctx->prof_events.size()) {
        hipEvent_t e0 = ctx->prof_events[2 * ctx->prof_used], e1 = ctx->prof_events[2 * ctx->prof_used + 1];
        ctx->prof_used++;
        hipExtLaunchKernelGGL(kernel, grid, block, (unsigned)lds, ctx->stream, e0, e1, 0, args...);
    } else {
        hipLaunchKernelGGL(kernel, grid, block, (unsigned)lds, ctx->stream, args...);
    }
}

#ifdef __HIPCC__
// v as an fp16 pair: hi = f16(v), lo = f16(v - hi).  v is first hidden from the optimizer: when it can see the
// product that made v, it fuses that product into each conversion separately (a fused convert rounds once, a
// plain one twice) and the hi that lo was taken against is then not always the hi that is stored.
__device__ __forceinline__ void skn_split_hilo(float v, _Float16& hi, _Float16& lo) {
    asm("" : "+v"(v));
    hi = (_Float16)v;
    lo = (_Float16)(v - (float)hi);
}
#endif

// the three formats with tuned kernels (and the only ones the decoder's embedding lookup reads)
static inline bool skn_is_core_quant(int t) { return t == SKN_TYPE_Q8_0 || t == SKN_TYPE_Q4_K || t == SKN_TYPE_Q6_K; }
// every format the library computes with
static inline bool skn_is_quant(int t) {
    return skn_is_core_quant(t) || t == SKN_TYPE_Q4_0 || t == SKN_TYPE_Q4_1 || t == SKN_TYPE_Q5_0 || t == SKN_TYPE_Q5_1 ||
           t == SKN_TYPE_Q2_K || t == SKN_TYPE_Q5_K || t == SKN_TYPE_F32 || t == SKN_TYPE_F16 || t == SKN_TYPE_BF16 ||
           t == SKN_TYPE_Q3_K || t == SKN_TYPE_Q8_K || t == SKN_TYPE_IQ4_NL || t == SKN_TYPE_IQ4_XS ||
           t == SKN_TYPE_TQ1_0 || t == SKN_TYPE_TQ2_0;
}
int skn_dequant_other(skn_ctx* ctx, int ggml_type, const uint8_t* w, int64_t n_elems, float* out);
int skn_matvec_other(skn_ctx* ctx, int ggml_type, const uint8_t* w, int n, int k, const float* x, float* y);
// Q4_K GEMM of one activation matrix [m, k] against up to three weight matrices [n_i, k] in one launch:
// c_i[m, n_i] (+)= a * w_i^T.  The activation rows are bf16 (as skn_gemm_q takes them), or fp32 that the GEMM's
// preparation pass rounds to bf16 itself -- optionally after the RMSNorm (weights b) that precedes the GEMM in
// a transformer block, with the arithmetic of the separate row-wise kernel.
enum { SKN_SRC_BF16 = 0, SKN_SRC_F32 = 1, SKN_SRC_RMSNORM = 2 };
struct skn_gemm_src {
    int kind;
    const void* a;
    const void* b;
    float eps;  // SKN_SRC_RMSNORM
};
struct skn_gemm_seg {
    const void* w;
    int n;
    float* c;
    int accumulate;  // c += instead of c =
};
// swiglu_pair: segs[0], segs[1] are the gate and up matrices of a SwiGLU; silu(gate) * up goes to segs[0].c ([m, n])
int skn_gemm_q4k_multi(skn_ctx* ctx, const skn_gemm_seg* segs, int nseg, int k, const skn_gemm_src& src, int m,
                       bool swiglu_pair = false);
int skn_weights_hilo_frag(skn_ctx* ctx, int ggml_type, const uint8_t* w, int n, int k, void* bfrag);
// The general GEMM path with weights expanded beforehand (skn_gemm_expand): one activation pass, then one launch per
// matrix; seg.w is the expanded copy (skn_gemm_expanded_size bytes).
size_t skn_gemm_expanded_size(int n, int k);
int skn_gemm_expanded_multi(skn_ctx* ctx, const skn_gemm_seg* segs, int nseg, int k, const skn_gemm_src& src, int m);

// ---- device helpers --------------------------------------------------------------------------------

constexpr int kWave = 64;

__device__ __forceinline__ float h2f_bits(uint32_t bits16) {
    return __half2float(__ushort_as_half((unsigned short)bits16));
}

// sin and cos of the rotary angle pos * base^(-e / head_dim) for the element pair (e, e + 1).  The angle is formed and
// reduced modulo 2 pi in double: in fp32 its rounding alone is pos * 2^-24 radians, which at a few hundred positions
// already shows in the small outputs of a rotated pair.
__device__ __forceinline__ void skn_rope_sincos_freq(int pos, double inv_freq, float* sn, float* cs) {
    const double theta = (double)pos * inv_freq;
    const double turns = rint(theta * 0.15915494309189535);  // 1 / (2 pi)
    const float r = (float)fma(-turns, 6.283185307179586, theta);
    sincosf(r, sn, cs);
}

__device__ __forceinline__ void skn_rope_sincos(int pos, int e, int head_dim, double log2_base, float* sn, float* cs) {
    const double theta = (double)pos * exp2(-(double)e / (double)head_dim * log2_base);
    const double turns = rint(theta * 0.15915494309189535);  // 1 / (2 pi)
    const float r = (float)fma(-turns, 6.283185307179586, theta);
    sincosf(r, sn, cs);
}

// Sum over the 64 lanes of a wavefront; every lane returns the total.
// Steps 1-4 stay inside a 16-lane row and use DPP lane permutations; the two cross-row steps read the
// four row totals back through scalar registers.
__device__ __forceinline__ float wave_sum(float v) {
    int i;
    i = __builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
    v += __int_as_float(i);
    i = __builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
    v += __int_as_float(i);
    i = __builtin_amdgcn_mov_dpp(__float_as_int(v), 0x141, 0xF, 0xF, true);  // row_half_mirror
    v += __int_as_float(i);
    i = __builtin_amdgcn_mov_dpp(__float_as_int(v), 0x140, 0xF, 0xF, true);  // row_mirror
    v += __int_as_float(i);
    float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return (r0 + r1) + (r2 + r3);
}

__device__ __forceinline__ float wave_max(float v) {
    int i;
    i = __builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xF, 0xF, true);
    v = fmaxf(v, __int_as_float(i));
    i = __builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xF, 0xF, true);
    v = fmaxf(v, __int_as_float(i));
    i = __builtin_amdgcn_mov_dpp(__float_as_int(v), 0x141, 0xF, 0xF, true);
    v = fmaxf(v, __int_as_float(i));
    i = __builtin_amdgcn_mov_dpp(__float_as_int(v), 0x140, 0xF, 0xF, true);
    v = fmaxf(v, __int_as_float(i));
    float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

// Sum over each aligned group of 16 lanes (one DPP row); every lane of the group returns its group's total.
__device__ __forceinline__ float row16_sum(float v) {
    int i;
    i = __builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xF, 0xF, true);
    v += __int_as_float(i);
    i = __builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xF, 0xF, true);
    v += __int_as_float(i);
    i = __builtin_amdgcn_mov_dpp(__float_as_int(v), 0x141, 0xF, 0xF, true);
    v += __int_as_float(i);
    i = __builtin_amdgcn_mov_dpp(__float_as_int(v), 0x140, 0xF, 0xF, true);
    v += __int_as_float(i);
    return v;
}

// Little-endian loads from addresses that are only 2-byte (or 1-byte) aligned.
__device__ __forceinline__ uint32_t load_u32_a2(const uint8_t* p) {
    const uint16_t* q = reinterpret_cast<const uint16_t*>(p);
    return (uint32_t)q[0] | ((uint32_t)q[1] << 16);
}
__device__ __forceinline__ uint32_t load_u16_a2(const uint8_t* p) {
    return *reinterpret_cast<const uint16_t*>(p);
}
