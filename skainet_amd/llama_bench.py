"""7B-shaped Q4_K decode throughput: 512-token random prompt, then 128 greedy steps, batch 1."""
from __future__ import annotations

import time

import numpy as np

from . import llama


def run(ctx, prompt_len=512, steps=128, seed=11, share_layers=False, matrix_type=None, matrix_types=None):
    """matrix_type: a ggml type id for the seven matrices of every layer instead of Q4_K; matrix_types: per-matrix
    types as llama.Config takes them (e.g. {"l0.wv": 14})."""
    types = {} if matrix_type is None else {m: matrix_type for m in ("wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down")}
    types.update(matrix_types or {})
    cfg = llama.Config(max_tokens=1024, matrix_types=types)
    t0 = time.perf_counter()
    model = llama.LlamaModel(ctx, cfg, seed=seed, share_layers=share_layers)
    build_s = time.perf_counter() - t0
    prompt = np.random.default_rng(seed).integers(0, cfg.vocab, size=prompt_len).tolist()
    t0 = time.perf_counter()
    first = model.prefill(prompt)
    prefill_s = time.perf_counter() - t0
    model.decode(first, 4)  # captures the step graph; not timed
    model.reset()
    t0 = time.perf_counter()
    first = model.prefill(prompt)
    ctx.sync()
    prefill_s = time.perf_counter() - t0
    t0 = time.perf_counter()
    toks = model.decode(first, steps)
    ctx.sync()
    decode_s = time.perf_counter() - t0
    wbytes = model.weight_bytes_per_token()
    kv_bytes = cfg.n_layer * cfg.hidden * 2 * 2 * (prompt_len + steps / 2.0)
    out = {
        "decode_tok_s": round(steps / decode_s, 2),
        "ms_per_token": round(decode_s / steps * 1e3, 4),
        "prefill_tok_s": round(prompt_len / prefill_s, 1),
        "prefill_ms": round(prefill_s * 1e3, 2),
        "weight_bytes_per_token": wbytes,
        "hbm_floor_tok_s": round(8.0e12 / (wbytes + kv_bytes), 1),
        "frac_of_hbm_floor": round((steps / decode_s) / (8.0e12 / (wbytes + kv_bytes)), 4),
        "prompt_len": prompt_len,
        "steps": steps,
        "distinct_weight_layers": 1 if share_layers else cfg.n_layer,
        "weights_build_s": round(build_s, 1),
        "tokens_head": toks[:8],
    }
    model.free()
    return out
