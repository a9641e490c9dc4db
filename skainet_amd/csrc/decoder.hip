// Llama-style decoder over the quantized kernels (placeholder entry points until the decoder lands).
#include "kv.h"

extern "C" {
int skn_llama_create(skn_ctx* ctx, const skn_llama_config*, const skn_llama_weights*, skn_llama** out) {
    if (out) *out = nullptr;
    return skn_fail(ctx, SKN_ERR_STATE, "skn_llama_create: decoder not built");
}
int skn_llama_free(skn_ctx* ctx, skn_llama*) { return skn_fail(ctx, SKN_ERR_STATE, "decoder not built"); }
int skn_llama_reset(skn_ctx* ctx, skn_llama*) { return skn_fail(ctx, SKN_ERR_STATE, "decoder not built"); }
int skn_llama_prefill(skn_ctx* ctx, skn_llama*, const int32_t*, int, int32_t*) {
    return skn_fail(ctx, SKN_ERR_STATE, "decoder not built");
}
int skn_llama_decode(skn_ctx* ctx, skn_llama*, int32_t, int, int32_t*) {
    return skn_fail(ctx, SKN_ERR_STATE, "decoder not built");
}
int skn_llama_logits(skn_ctx* ctx, skn_llama*, const float**) { return skn_fail(ctx, SKN_ERR_STATE, "decoder not built"); }
}
