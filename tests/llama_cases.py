"""The conditioned decoder models shared by the CPU sensitivity test and the GPU parity tests.

Weights come from llama.conditioned_weights (zero-centred, a power-of-two scale per matrix), pages hold 16 tokens so
that a run of 44 tokens crosses two page boundaries."""
from skainet_amd import llama

_BASE = dict(n_layer=2, hidden=512, ffn=768, n_head=4, head_dim=128, vocab=512, max_tokens=96, page_tokens=16)

CASES = {
    # every layer matrix Q4_K (the fused Q4_K kernels), Q4_K embedding, Q6_K head: the benchmark's format mix
    "q4_k": llama.Config(**_BASE),
    # grouped-query attention: two query heads per cached head, and one cached head for all four
    "q4_k_kv2": llama.Config(**_BASE, n_kv_head=2),
    "q4_k_kv1": llama.Config(**_BASE, n_kv_head=1),
    # the zero-centred formats beside Q4_K, every group once in another format
    "mixed": llama.Config(**_BASE, n_kv_head=2, matrix_types={"l0.wq": 8, "l0.wk": 8, "l0.wv": 14, "l0.w_down": 14,
                                                              "l1.wo": 8, "l1.w_gate": 2, "l1.w_up": 2, "l1.wv": 6}),
    "q8_0": llama.Config(**_BASE, type_attn=8, type_ffn=8, type_embd=8),
    "q6_k": llama.Config(**_BASE, n_kv_head=2, type_attn=14, type_ffn=14),
}
SEED = 3
DECODE_TOL = 2e-3   # the decoder tests' bound for two layers (1e-3 per operation, sqrt(2 n) for n layers)
PROMPT_TOL = 5e-3   # prompt pass: bf16 activations in every projection


def logit_err(got, want):
    """max |got - want| / max |want|.  The logits of these models are centred on zero, so some are always within
    rounding of it and an error relative to each logit's own size measures nothing but those; and the cached keys
    and values are fp16, so a difference in the last bit of an fp32 key flips an fp16 rounding now and then, which
    moves every later logit by about 1e-4 of the largest (test_oracle_llama_sensitivity.py measures both)."""
    import numpy as np

    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    return float(np.max(np.abs(got - want)) / np.max(np.abs(want)))


def tokens(n, vocab, seed=1):
    import numpy as np

    return np.random.default_rng(seed).integers(0, vocab, size=n).tolist()
