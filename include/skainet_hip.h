/*
 * libskainet_hip -- C ABI of the MI355X (gfx950) quantized-inference hot path for sk-ai-net/skainet.
 *
 * The reference has no native boundary of its own (it is pure Kotlin); these entry points are what a
 * Kotlin/Native cinterop .def or a JVM Panama FFM binding would bind so that a device-backed tensor can
 * sit behind the reference's existing seams.  Each declaration cites the reference interface it serves.
 *
 * Conventions
 *   - Every function returns SKN_OK (0) or a negative SKN_ERR_* code; nothing throws or aborts across the
 *     boundary.  skn_last_error() gives the message of the last failure on that context.
 *   - `dev` pointers are device addresses (from skn_malloc, or any HIP allocation of the same process);
 *     `host` pointers are ordinary host memory borrowed for the duration of the call.
 *   - ggml type ids are the reference's GGMLQuantizationType values
 *     (gguf/src/commonMain/kotlin/sk/ai/net/gguf/Constants.kt:14-46): F32 0, F16 1, Q8_0 8, Q4_K 12, Q6_K 14.
 *   - Weights are [n, k] = [out, in] as in the reference's Linear (core/.../nn/Linear.kt:26-28): n rows, each
 *     k / block consecutive GGUF blocks, rows contiguous -- exactly the bytes GGUFReader hands out for a
 *     quantized tensor (gguf/.../GGUFReader.kt:354-373).
 *   - One HIP stream per context; compute calls are asynchronous on it; skn_sync / skn_download wait.
 *     Calls on one context must be serialised by the caller (the reference is single-threaded throughout).
 */
#ifndef SKAINET_HIP_H
#define SKAINET_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SKN_ABI_VERSION 2

#define SKN_OK 0
#define SKN_ERR_ARG (-1)    /* null pointer, negative size, bad handle */
#define SKN_ERR_TYPE (-2)   /* ggml type id not on this path */
#define SKN_ERR_SHAPE (-3)  /* row not a block multiple / operands do not align */
#define SKN_ERR_OOM (-4)    /* device or host allocation failed */
#define SKN_ERR_HIP (-5)    /* a HIP runtime call failed */
#define SKN_ERR_RANGE (-6)  /* sequence id / token range outside the cache */
#define SKN_ERR_POOL (-7)   /* KV page pool exhausted or sequence full */
#define SKN_ERR_STATE (-8)  /* call not valid in the current state */

#define SKN_TYPE_F32 0
#define SKN_TYPE_F16 1
#define SKN_TYPE_Q4_0 2
#define SKN_TYPE_Q4_1 3
#define SKN_TYPE_Q5_0 6
#define SKN_TYPE_Q5_1 7
#define SKN_TYPE_Q8_0 8
#define SKN_TYPE_Q2_K 10
#define SKN_TYPE_Q3_K 11
#define SKN_TYPE_Q4_K 12
#define SKN_TYPE_Q5_K 13
#define SKN_TYPE_Q6_K 14
#define SKN_TYPE_Q8_K 15
#define SKN_TYPE_IQ4_NL 20
#define SKN_TYPE_IQ4_XS 23
#define SKN_TYPE_BF16 30
#define SKN_TYPE_TQ1_0 34
#define SKN_TYPE_TQ2_0 35

typedef struct skn_ctx skn_ctx;
typedef struct skn_kv skn_kv;
typedef struct skn_llama skn_llama;

/* ---- lifetime, errors -------------------------------------------------------------------------- */

int skn_abi_version(void);
/* Creates a context on HIP device `device` with its own stream.  (No reference counterpart: reference
 * tensors are garbage-collected host objects; a Kotlin wrapper would be AutoCloseable around this.) */
int skn_init(int device, skn_ctx** out);
void skn_shutdown(skn_ctx* ctx);
/* Message of the last error on `ctx` (or of the last context-less failure when ctx is NULL). */
const char* skn_last_error(skn_ctx* ctx);
const char* skn_status_string(int code);
/* Device facts for reports: name, compute units, total memory. */
int skn_device_info(skn_ctx* ctx, char* name, size_t name_len, int* compute_units, size_t* total_bytes);

/* ---- format table -------------------------------------------------------------------------------- */

/* GGML_QUANT_SIZES lookup (gguf/.../Constants.kt:58-90): elements and bytes per block, for every type id of
 * that table (the ids of gguf/.../Constants.kt:14-46).  The kernels compute with the SKN_TYPE_* ids above. */
int skn_type_block(int ggml_type, int* block_elems, int* block_bytes);
/* quantShapeToByteShape on the last axis (gguf/.../Quants.kt:10-20): bytes of a row of k elements, or
 * SKN_ERR_SHAPE when k is not a block multiple, SKN_ERR_TYPE for an unknown type. */
int64_t skn_row_bytes(int ggml_type, int64_t k);

/* ---- device memory ------------------------------------------------------------------------------- */

/* Where the bytes of ReaderTensor.data (gguf/.../GGUFReader.kt:35-44,370-395) go to live on the device. */
int skn_malloc(skn_ctx* ctx, size_t bytes, void** dev);
int skn_free(skn_ctx* ctx, void* dev);
int skn_upload(skn_ctx* ctx, void* dev, const void* host, size_t bytes);
int skn_download(skn_ctx* ctx, void* host, const void* dev, size_t bytes);
int skn_memset(skn_ctx* ctx, void* dev, int byte_value, size_t bytes);
/* Device-to-device copy by a streaming kernel on the context's stream (ranges must not overlap). */
int skn_copy(skn_ctx* ctx, void* dst_dev, const void* src_dev, size_t bytes);
int skn_sync(skn_ctx* ctx);
/* Adopt a caller-owned hipStream_t (NULL restores the context's own stream). */
int skn_set_stream(skn_ctx* ctx, void* hip_stream);
/* Launch-shape tuning knobs, 0 = library default: "q4k.waves" (wavefronts per workgroup of the Q4_K matvec),
 * "q4k.rows" (rows per wavefront: 1, 2 or 4), "attn.splits" (context splits of decode attention),
 * "llama.graph" (1 = replay a captured HIP graph per decode step, the default; 0 = launch every kernel; a captured
 * step is dropped and captured again after any change of an option or of the stream),
 * "llama.fused" (1 = fused per-layer kernels in the decode step, the default: for every group of matrices whose
 * formats have one -- Q4_K, Q5_K, Q4_0, Q4_1, Q5_0, Q5_1, IQ4_NL, IQ4_XS, Q6_K, Q8_0, Q2_K, Q3_K, Q8_K, TQ1_0, TQ2_0), "llama.expand_weights" (1 = the prompt pass of a decoder keeps an expanded
 * copy, see skn_gemm_expand, of every layer matrix that is not Q4_K, made at the first prompt: 4 bytes per weight of
 * device memory on top of the blocks; 0 = the default, expand per call), "gemm.tile" (0 = choose, 1 = 64-row tiles,
 * 2 = 128-row tiles of the Q4_K GEMM), "matvec.stage" (kernel family of the further formats' matvec: 1 = the
 * default -- the Q4_K kernel's lane map for Q5_K / Q4_0 / Q4_1 / Q5_0 / Q5_1 / IQ4_NL / IQ4_XS / Q8_K, the Q6_K kernel's for
 * Q2_K / Q3_K / TQ2_0, its own for TQ1_0, rows staged through LDS for what is left with 4-byte-multiple blocks; 2 = staged rows for all
 * formats with such blocks; 0 = direct reads).  The knobs exist for
 * measurements and tests; every setting computes the same results to the tolerance of the operation. */
int skn_set_option(skn_ctx* ctx, const char* key, int value);
/* Counters of a context, for tests and reports: "launches" (kernel launches issued or recorded into a graph so far),
 * "graph.captures" (decode-step graphs captured so far), "llama.expanded_bytes" (device bytes that the
 * decoders of this context hold in expanded weight copies, see "llama.expand_weights"), "profiler.attached" (1 when a rocprofiler tool library is
 * loaded into the process: "llama.graph" is then 0 and cannot be set, every decode step is launched kernel by kernel). */
int skn_get_stat(skn_ctx* ctx, const char* key, int64_t* value);
/* HIP-event stopwatch on the context's stream: start, enqueue work, stop -> elapsed milliseconds. */
int skn_timer_start(skn_ctx* ctx);
int skn_timer_stop(skn_ctx* ctx, float* elapsed_ms);
/* Per-launch kernel timing: between start and stop each kernel launched on this context carries its own
 * start/stop HIP events (dispatch begin/end timestamps); stop waits for the stream and returns the summed
 * kernel durations and the number of launches timed (at most max_launches). */
int skn_prof_start(skn_ctx* ctx, int max_launches);
int skn_prof_stop(skn_ctx* ctx, double* kernel_ms_total, int* launches);

/* ---- dequantization ------------------------------------------------------------------------------ */

/* The dequantizer the reference leaves as a TODO (gguf/.../Quants.kt:8): n_elems consecutive elements
 * (a block multiple) of `ggml_type` at `w_dev` -> fp32 at `out_dev`.  Bit-exact with the ggml formulas.
 * Types: every SKN_TYPE_* id (F32 / F16 / BF16 are widened or copied). */
int skn_dequant(skn_ctx* ctx, int ggml_type, const void* w_dev, int64_t n_elems, float* out_dev);

/* ---- quantized matvec / GEMM ---------------------------------------------------------------------- */

/* y[n] = sum_k deq(W)[n,k] * x[k]: Linear.forward's `input.matmul(weight.t())` for a rank-1 input
 * (core/.../nn/Linear.kt:43-49 -> core/.../impl/DoublesTensor.kt:255-264), without materialising t().
 * x fp32 [k], y fp32 [n].  Any SKN_TYPE_* weight type; Q4_K, Q8_0 and Q6_K have the tuned kernels. */
int skn_matvec_q(skn_ctx* ctx, int ggml_type, const void* w_dev, int n, int k, const float* x_dev, float* y_dev);
/* C[m,n] = sum_k A[m,k] * deq(W)[n,k]: the rank-2 case (core/.../impl/DoublesTensor.kt:267-279).
 * A bf16 bits [m,k] row-major, C fp32 [m,n] row-major. */
int skn_gemm_q(skn_ctx* ctx, int ggml_type, const void* w_dev, int n, int k, const uint16_t* a_bf16_dev, int m,
               float* c_dev);
/* The same product (core/.../impl/DoublesTensor.kt:267-279) with the weight pass of the formats other than Q4_K done
 * once instead of per call.  For those formats skn_gemm_q first rewrites W as an fp16 pair per weight in matrix-core
 * operand order (4 bytes per weight, rows padded to a multiple of 64); a caller that multiplies with the same W
 * again and has the memory keeps that copy: skn_gemm_expanded_bytes gives its size, skn_gemm_expand fills a device
 * buffer of that size (16-byte aligned) from the blocks, skn_gemm_expanded multiplies with it -- the results are
 * those of skn_gemm_q bit for bit.  Any SKN_TYPE_* weight type; k a multiple of 64. */
int skn_gemm_expanded_bytes(skn_ctx* ctx, int ggml_type, int n, int k, size_t* bytes_out);
int skn_gemm_expand(skn_ctx* ctx, int ggml_type, const void* w_dev, int n, int k, void* expanded_dev);
int skn_gemm_expanded(skn_ctx* ctx, const void* expanded_dev, int n, int k, const uint16_t* a_bf16_dev, int m,
                      float* c_dev);

/* ---- paged KV cache -------------------------------------------------------------------------------- */

/* No reference counterpart (the reference has no sequences or attention).  A cache holds fp16 K and V rows of
 * n_head * head_dim values per token for n_seq sequences, in device pages of page_tokens tokens drawn on
 * demand from a pool sized for n_seq * ceil(max_tokens / page_tokens) pages. */
int skn_kv_create(skn_ctx* ctx, int n_seq, int n_head, int head_dim, int page_tokens, int max_tokens, skn_kv** out);
int skn_kv_free(skn_ctx* ctx, skn_kv* kv);
/* Forget the tokens of one sequence (seq >= 0) or of all (seq = -1); pages return to the pool. */
int skn_kv_reset(skn_ctx* ctx, skn_kv* kv, int seq);
/* Current token count of a sequence, or a negative error code. */
int skn_kv_len(skn_ctx* ctx, skn_kv* kv, int seq);
/* Append one token for each of n listed sequences: k/v fp16 bits [n][n_head][head_dim] on the device,
 * seq_ids on the host (a sequence may be listed more than once; its tokens land in list order). */
int skn_kv_append(skn_ctx* ctx, skn_kv* kv, const uint16_t* k_dev, const uint16_t* v_dev, const int32_t* seq_ids_host,
                  int n);
/* Append n_tokens consecutive tokens to one sequence: k/v fp16 bits [n_tokens][n_head][head_dim]. */
int skn_kv_append_run(skn_ctx* ctx, skn_kv* kv, int seq, const uint16_t* k_dev, const uint16_t* v_dev, int n_tokens);
/* Copy tokens [t0, t1) of a sequence out, token-major [t1-t0][n_head][head_dim] fp16 bits. */
int skn_kv_gather(skn_ctx* ctx, skn_kv* kv, int seq, int t0, int t1, uint16_t* k_out_dev, uint16_t* v_out_dev);

/* out[s,h,:] = softmax(q[s,h,:] . K[s,0:n,h,:]^T * scale) . V[s,0:n,h,:] for every sequence and head.
 * q/out fp32 [n_seq][n_head][head_dim] on the device; n_ctx_host[s] = tokens to attend (NULL = all cached). */
int skn_attn_decode(skn_ctx* ctx, skn_kv* kv, const float* q_dev, const int32_t* n_ctx_host, float scale,
                    float* out_dev);
/* skn_attn_decode over all cached tokens of every sequence, for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * The split partials and split counters live in a fixed array inside the library's device image (4 MiB + 16 KiB per
 * GPU, held until the process ends) instead of hipMalloc'd scratch; the call allocates and frees nothing.
 * Limits: n_seq * n_head <= 4096, and n_seq * n_head * splits * (head_dim + 2) * 4 bytes <= 4 MiB -- SKN_ERR_SHAPE
 * beyond them.  Every call on a GPU shares that GPU's array: calls that overlap on one GPU (two contexts, two
 * streams) race; serialise them. */
int skn_attn_decode_static(skn_ctx* ctx, skn_kv* kv, const float* q_dev, float scale, float* out_dev);
/* The same attention for the last n_queries tokens of one sequence at once (prompt processing), causal:
 * out[t,h,:] = softmax(q[t,h,:] . K[0:m_t,h,:]^T * scale) . V[0:m_t,h,:] with m_t = len - n_queries + t + 1.
 * q/out fp32 [n_queries][n_head][head_dim] on the device, 16-byte aligned; head_dim 64 or 128.  No reference
 * counterpart, like the cache itself. */
int skn_attn_prefill(skn_ctx* ctx, skn_kv* kv, int seq, const float* q_dev, int n_queries, float scale, float* out_dev);

/* ---- decoder glue (fp32, device pointers) ------------------------------------------------------------ */

/* y = x / sqrt(mean(x^2) + eps) * w, row-wise over `rows` rows of n. */
int skn_rmsnorm(skn_ctx* ctx, const float* x_dev, const float* w_dev, int rows, int n, float eps, float* y_dev);
/* Rotary embedding in place on [rows][n_head][head_dim]; row r is at position pos0 + r; interleaved pairs
 * (2i, 2i+1), angle = pos * base^(-2i/head_dim). */
int skn_rope(skn_ctx* ctx, float* x_dev, int rows, int n_head, int head_dim, int pos0, float base);
/* out = silu(gate) * up elementwise. */
int skn_swiglu(skn_ctx* ctx, const float* gate_dev, const float* up_dev, int64_t n, float* out_dev);
/* out = max(x, 0) elementwise, the reference's Tensor.relu (core/.../impl/DoublesTensor.kt:389-390: `if (elem > 0)
 * elem else 0.0`, so a NaN gives 0), which its ReLU module applies between Linear layers
 * (core/.../nn/activations/relu.kt:7-12).  out may be x. */
int skn_relu(skn_ctx* ctx, const float* x_dev, int64_t n, float* out_dev);
/* y += x elementwise. */
int skn_add_inplace(skn_ctx* ctx, float* y_dev, const float* x_dev, int64_t n);
/* Index of the first maximum of x[0:n] -> *index_dev (int32 on the device); the reference's inline scan
 * (samples/mnist-mlp-cli/src/jvmMain/kotlin/sk/ai/net/samples/mnist/mlp/Main.kt:269-278) keeps the first too. */
int skn_argmax(skn_ctx* ctx, const float* x_dev, int n, int32_t* index_dev);
/* fp32 -> fp16 / bf16 bits and back, elementwise (round to nearest even). */
int skn_f32_to_f16(skn_ctx* ctx, const float* x_dev, int64_t n, uint16_t* out_dev);
int skn_f32_to_bf16(skn_ctx* ctx, const float* x_dev, int64_t n, uint16_t* out_dev);

/* ---- Llama-style decoder (7B-shaped Q4_K decode) ------------------------------------------------------ */

typedef struct skn_llama_config {
    int32_t n_layer;     /* 32 */
    int32_t hidden;      /* 4096 */
    int32_t ffn;         /* 11008 */
    int32_t n_head;      /* 32 */
    int32_t head_dim;    /* 128 */
    int32_t vocab;       /* 32000 */
    int32_t max_tokens;  /* KV capacity of the single sequence */
    int32_t page_tokens; /* 256 */
    float rope_base;     /* 10000 */
    float rms_eps;       /* 1e-5 */
    int32_t n_kv_head;   /* heads of the K / V projections and of the cache: a divisor of n_head (grouped-query
                            attention), or 0 for n_head */
} skn_llama_config;

/* Per-layer weights, all device pointers into GGUF block data ([out, in] rows) or fp32 norm vectors. */
typedef struct skn_llama_layer {
    const void* wq; const void* wo;                                  /* [hidden, hidden] */
    const void* wk; const void* wv;                                  /* [n_kv_head * head_dim, hidden] */
    const void* w_gate; const void* w_up;                            /* [ffn, hidden] */
    const void* w_down;                                              /* [hidden, ffn] */
    const float* attn_norm; const float* ffn_norm;                   /* [hidden] */
    /* ggml type id of each matrix (files quantized with a mix give some matrices of a layer more bits) */
    int32_t type_q; int32_t type_k; int32_t type_v; int32_t type_o;
    int32_t type_gate; int32_t type_up; int32_t type_down;
} skn_llama_layer;

typedef struct skn_llama_weights {
    const void* tok_embd;    /* [vocab, hidden], ggml type `type_embd` */
    const float* out_norm;   /* [hidden] */
    const void* out_head;    /* [vocab, hidden], ggml type `type_head` */
    int32_t type_embd; int32_t type_head;
    const skn_llama_layer* layers; /* host array of n_layer entries (copied) */
} skn_llama_weights;

/* The module graph the reference would express as nested Module.forward calls (core/.../nn/Module.kt:6-16,
 * core/.../nn/topology/MLP.kt:13-19) for a Llama block stack; weights stay owned by the caller.  Every layer matrix and
 * norm vector must be 16-byte aligned on the device (what skn_malloc returns is). */
int skn_llama_create(skn_ctx* ctx, const skn_llama_config* cfg, const skn_llama_weights* w, skn_llama** out);
int skn_llama_free(skn_ctx* ctx, skn_llama* m);
int skn_llama_reset(skn_ctx* ctx, skn_llama* m);
/* Runs n_tokens prompt tokens (host ids) through the model with batched GEMMs, filling the KV cache;
 * logits of the last token (fp32 [vocab]) stay on the device, *next_token_host receives their argmax. */
int skn_llama_prefill(skn_ctx* ctx, skn_llama* m, const int32_t* tokens_host, int n_tokens, int32_t* next_token_host);
/* Greedy decode: feeds `first_token`, then its own argmax, for n_steps steps; tokens_out_host[i] is the token
 * produced by step i.  One captured HIP graph per step shape is replayed. */
int skn_llama_decode(skn_ctx* ctx, skn_llama* m, int32_t first_token, int n_steps, int32_t* tokens_out_host);
/* Device pointer to the fp32 [vocab] logits of the last processed token. */
int skn_llama_logits(skn_ctx* ctx, skn_llama* m, const float** logits_dev);

/* ---- test hook (not part of the surface a binding needs) ------------------------------------------------ */

/* One launch of the fused matvec the decoder uses, so that tests can hold each fused form against the CPU oracle as an
 * operation of its own: up to three [rows_i, k] matrices of one type stacked along the output, optional RMSNorm of x
 * (norm_w_dev, eps), and an epilogue: 0 store y, 1 y +=, 2 y[i] = silu(w0 row i . x) * (w1 row i . x), 3 rotary
 * embedding of q (rows0, to y as fp32) and k (rows1) with k and v (rows2) stored as fp16 at the end of sequence 0 of the
 * one-sequence cache `kv` (its position is written to *pos_dev, a device int the caller provides).  No reference
 * counterpart.  Types: Q4_K, Q5_K, Q4_0, Q4_1, Q5_0, Q5_1, IQ4_NL, IQ4_XS, Q6_K, Q8_0, Q2_K, Q3_K, Q8_K, TQ1_0, TQ2_0; k a multiple of 256,
 * at most 16384. */
int skn_test_fused_matvec(skn_ctx* ctx, int ggml_type, int epi, const void* w0, int rows0, const void* w1, int rows1,
                          const void* w2, int rows2, int k, const float* x_dev, const float* norm_w_dev, float eps,
                          float* y_dev, skn_kv* kv, int32_t* pos_dev, float rope_base);
/* The Q4_K matvec of skn_matvec_q for a row of three steps (8192 < k <= 12288, one row per wavefront) run with the
 * kernel's measuring build: y as usual, and eight 64-bit words per row (= per wavefront) in stamps_dev -- the 100 MHz
 * wall clock at the wavefront's start, after its first requests are issued, after its stores of x, after the
 * barrier, after each of the three steps, and (XCC_ID << 32 | HW_ID).  For `bench.py --mode timeline`.  No
 * reference counterpart. */
int skn_test_matvec_q4k_stamps(skn_ctx* ctx, const void* w_dev, int n, int k, const float* x_dev, float* y_dev,
                               uint64_t* stamps_dev);
/* Two measurements of the machine that the kernel designs lean on (`bench.py --mode machine`); no reference
 * counterpart.  (1) Nanoseconds per v_mfma_f32_32x32x16_f16 and SIMD when every matrix instruction is followed by
 * valu_per_mfma (0, 2, 4, 6, 7, 8 or 12) independent vector instructions, at one or two wavefronts per SIMD;
 * scratch_dev: 512 KiB of device memory.  (2) GB/s per compute unit at which 1 KiB operand fragments (one 16-byte load
 * per lane, eight in flight per wavefront, eight wavefronts per compute unit) arrive in registers when `share` (1, 2, 4
 * or 8) wavefronts of a workgroup read the same fragments; data_dev: data_mib MiB of device memory, flag_dev: one
 * device word. */
int skn_test_mfma_valu_overlap(skn_ctx* ctx, int waves_per_simd, int valu_per_mfma, float* scratch_dev, double* ns_out);
int skn_test_fragment_delivery(skn_ctx* ctx, int share, const void* data_dev, int data_mib, unsigned* flag_dev,
                               double* gbs_out);
/* Nanoseconds per k-step and SIMD (two wavefronts, eight matrix instructions) of a model of the Q4_K GEMM's inner loop
 * with some of its parts left out (`bench.py --mode machine`); parts, bit by bit: 1 nibble decode, 2 nibbles from LDS
 * and scale unpack, 4 activation fragments from memory, 8 header unpack per superblock, 16 accumulator rescale, 32 the
 * "- dmin * m" term; built: 0, 3, 4, 7, 15, 31, 47, 55, 59, 63.  data_dev: 64 MiB of device memory, scratch_dev:
 * 512 KiB.  No reference counterpart. */
int skn_test_q4k_gemm_loop(skn_ctx* ctx, int parts, const void* data_dev, float* scratch_dev, double* ns_out);

#ifdef __cplusplus
}
#endif
#endif /* SKAINET_HIP_H */
