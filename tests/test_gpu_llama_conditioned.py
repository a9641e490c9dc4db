"""Decoder parity on models whose logits depend on positions, cache contents and attention.

The models are tests/llama_cases.py's (zero-centred weights, attention scores of order one to ten);
tests/test_oracle_llama_sensitivity.py shows on the CPU that a dropped rotary embedding, a relative position off by
one, an attention that misses the newest token or sees only it, and a wrong cached head each move these logits by at
least ten tolerances at every step.  Here the HIP decoder runs them against the unmodified oracle: 44 decode steps
(pages of 16 tokens: two boundaries), a 41-token prompt followed by decode steps, grouped-query attention with two
and one cached heads, fused and separate kernels, captured graph and kernel-by-kernel launches.  Steps are fed
random tokens (teacher-forced), logits compared at every step as max |difference| / max |logit| (llama_cases.logit_err
says why not relative to each logit)."""
import numpy as np
import pytest

from llama_cases import CASES, DECODE_TOL, PROMPT_TOL, SEED, logit_err, tokens
from oracle.llama_oracle import OracleLlama
from skainet_amd import llama

pytestmark = pytest.mark.gpu

_ORACLE = {}


def _oracle_decode(case, n):
    """(tokens, logits per step) of the oracle, computed once per case."""
    key = (case, "decode", n)
    if key not in _ORACLE:
        cfg = CASES[case]
        ora = OracleLlama(cfg, llama.conditioned_weights(cfg, SEED))
        toks = tokens(n, cfg.vocab)
        out = []
        for t in toks:
            ora.step(t)
            out.append(ora.logits.copy())
        _ORACLE[key] = (toks, out)
    return _ORACLE[key]


def _oracle_prompt(case, n_prompt, n_steps):
    key = (case, "prompt", n_prompt, n_steps)
    if key not in _ORACLE:
        cfg = CASES[case]
        ora = OracleLlama(cfg, llama.conditioned_weights(cfg, SEED))
        prompt = tokens(n_prompt, cfg.vocab, seed=2)
        ora.prefill(prompt, bf16_gemm=True)
        first = ora.logits.copy()
        toks = tokens(n_steps, cfg.vocab, seed=4)
        out = []
        for t in toks:
            ora.step(t)
            out.append(ora.logits.copy())
        _ORACLE[key] = (prompt, first, toks, out)
    return _ORACLE[key]


class _Options:
    def __init__(self, hip, fused, graph):
        self.hip, self.fused, self.graph = hip, fused, graph

    def __enter__(self):
        self.hip.set_option("llama.fused", self.fused)
        self.hip.set_option("llama.graph", self.graph)

    def __exit__(self, *exc):
        self.hip.set_option("llama.fused", 1)
        self.hip.set_option("llama.graph", 1)


MODES = [(1, 1), (1, 0), (0, 1), (0, 0)]


@pytest.mark.parametrize("fused,graph", MODES)
@pytest.mark.parametrize("case", list(CASES))
def test_44_decode_steps_across_two_page_boundaries(hip, case, fused, graph):
    cfg = CASES[case]
    toks, want = _oracle_decode(case, 44)
    with _Options(hip, fused, graph):
        model = llama.LlamaModel(hip, cfg, weights=llama.conditioned_weights(cfg, SEED))
        worst = 0.0
        for i, t in enumerate(toks):
            model.decode(t, 1)
            err = logit_err(model.logits(), want[i])
            worst = max(worst, err)
            assert err <= DECODE_TOL, (case, fused, graph, i, err)
        print(f"{case} fused={fused} graph={graph}: worst logit error {worst:.2e}")
        model.free()


@pytest.mark.parametrize("case", ["q4_k", "q4_k_kv2", "q4_k_kv1", "mixed"])
def test_prompt_with_the_wide_tile_gemm_forced(hip, case):
    """The prompt's Q4_K products on 256 x 128 tiles, which the library otherwise picks from 129 rows on where they
    fill the device: the q, k, v group with one launch over three matrices (of 512, 256 or 128 columns with grouped
    K/V: tiles that end in another matrix's columns or past the last), the gate / up pair with SwiGLU in the store
    (768 columns: twelve tiles of 64 + 64), the output and down projections with the residual added."""
    cfg = CASES[case]
    prompt, first, toks, want = _oracle_prompt(case, 41, 12)
    hip.set_option("gemm.tile", 3)
    try:
        model = llama.LlamaModel(hip, cfg, weights=llama.conditioned_weights(cfg, SEED))
        model.prefill(prompt)
        err = logit_err(model.logits(), first)
        assert err <= PROMPT_TOL, (case, "prompt", err)
        for i, t in enumerate(toks[:4]):
            model.decode(t, 1)
            err = logit_err(model.logits(), want[i])
            assert err <= PROMPT_TOL, (case, i, err)
        model.free()
    finally:
        hip.set_option("gemm.tile", 0)


@pytest.mark.parametrize("fused,graph", [(1, 1), (0, 0)])
@pytest.mark.parametrize("case", list(CASES))
def test_41_token_prompt_then_decode_steps(hip, case, fused, graph):
    """The prompt's keys are rotated and stored by the prompt path (GEMMs, rotary + store kernel, prompt attention),
    the steps after it by the decode path: a position or cache-slot disagreement between the two shows in every
    later step's logits."""
    cfg = CASES[case]
    prompt, first, toks, want = _oracle_prompt(case, 41, 12)
    with _Options(hip, fused, graph):
        model = llama.LlamaModel(hip, cfg, weights=llama.conditioned_weights(cfg, SEED))
        model.prefill(prompt)
        err = logit_err(model.logits(), first)
        assert err <= PROMPT_TOL, (case, "prompt", err)
        worst = err
        for i, t in enumerate(toks):
            model.decode(t, 1)
            err = logit_err(model.logits(), want[i])
            worst = max(worst, err)
            assert err <= PROMPT_TOL, (case, fused, graph, i, err)
        print(f"{case} fused={fused} graph={graph}: worst logit error {worst:.2e}")
        model.free()


def test_several_steps_per_call_equal_one_step_per_call(hip):
    """skn_llama_decode with n steps feeds its own greedy tokens back: the same tokens and final logits as n calls."""
    cfg = CASES["q4_k_kv2"]
    w = llama.conditioned_weights(cfg, SEED)
    a = llama.LlamaModel(hip, cfg, weights=w)
    b = llama.LlamaModel(hip, cfg, weights=w)
    first = a.prefill([5, 6, 7])
    assert b.prefill([5, 6, 7]) == first
    many = a.decode(first, 40)
    tok, single = first, []
    for _ in range(40):
        tok = b.decode(tok, 1)[0]
        single.append(tok)
    assert many == single and len(set(many)) > 4  # (the greedy tokens of this model are not one token repeated)
    assert np.array_equal(a.logits(), b.logits())
    ora = OracleLlama(cfg, w)
    ora.prefill([5, 6, 7], bf16_gemm=True)
    tok = first
    for i in range(40):
        want = ora.step(tok)
        s = np.sort(ora.logits)
        if s[-1] - s[-2] <= 2 * PROMPT_TOL * np.abs(ora.logits).max():
            break
        assert many[i] == want, i
        tok = want
    a.free()
    b.free()


def test_hidden_4096_at_the_benchmark_length_matches_the_oracle_golden(hip, golden_dir):
    """Four distinct layers of the 7B model's width (hidden 4096, FFN 11008, 32 heads x 128, vocabulary 32000) on
    conditioned weights, 512-token prompt and 128 decode steps, against tests/golden/conditioned_4layer_512_128.npz
    (tests/golden/make_conditioned_golden.py: ten minutes of the CPU oracle).  Here the prompt GEMMs (M = 512), the
    prompt attention, the 2 -> 3 page boundary at 512 and the decode attention at contexts 513 to 640 all shape
    logits that the golden's own mutation record says move by at least 0.07 of the largest logit when the rotary
    embedding or the attention window is wrong.  Decode steps are fed the oracle's tokens.

    Tolerance: 5e-3 for two layers with bf16 prompt activations, times sqrt(4 / 2) for four: 7e-3 of the largest
    logit, for the prompt's last row and for every stored step (whose cache was written by the prompt path)."""
    import os

    gold = np.load(os.path.join(golden_dir, "conditioned_4layer_512_128.npz"))
    tol = PROMPT_TOL * np.sqrt(int(gold["n_layer"]) / 2)
    for m in ("no_rope", "pos_plus_one", "ctx_minus_one", "last_only"):
        assert float(gold[f"mutation_{m}_min"]) >= 9 * tol, m  # (recorded by the script that wrote the golden)
    stride = int(gold["stride"])
    cfg = llama.Config(n_layer=int(gold["n_layer"]), max_tokens=1024)
    model = llama.LlamaModel(hip, cfg, weights=llama.conditioned_weights(cfg, int(gold["seed"])))

    def check(tag, got_token):
        want, absmax = gold[f"{tag}_sample"].astype(np.float64), float(gold[f"{tag}_absmax"])
        err = float(np.max(np.abs(model.logits()[::stride].astype(np.float64) - want)) / absmax)
        assert err <= tol, (tag, err)
        if float(gold[f"{tag}_margin"]) > 2 * tol * absmax:
            assert got_token == int(gold[f"{tag}_argmax"]), tag
        return err

    errs = {"prefill": check("prefill", model.prefill(gold["prompt"].tolist()))}
    fed = [int(gold["first"])] + gold["tokens"].tolist()
    assert len(set(fed)) > 40  # (a golden whose greedy tokens repeat one token would say little)
    same = 0
    for i in range(128):
        tok = model.decode(fed[i], 1)[0]
        same += tok == fed[i + 1]
        if f"step{i}_sample" in gold.files:
            errs[f"step{i}"] = check(f"step{i}", tok)
    print("logit errors:", {k: f"{v:.2e}" for k, v in errs.items()}, "greedy tokens equal:", same, "of 128")
    assert same >= 120  # (steps whose top two logits are closer than the tolerance may differ)
    model.free()


@pytest.mark.parametrize("wide", [1, 2, 0])
@pytest.mark.parametrize("case,prompt_len", [("q4_k_kv2", 250), ("q4_k", 500), ("mixed", 500)])
def test_decode_across_the_split_boundaries_of_the_attention(hip, case, prompt_len, wide):
    """Contexts of 251 to 280 and 501 to 530 tokens: the decode attention goes from one workgroup per head to two and
    from two to four while the steps run (llama.attn_wide = 1: the splits' partials are merged by the output projection's
    staging; 0: by the attention kernel's last workgroup).  Prompt through the prompt path, thirty steps fed random
    tokens, every step's logits against the oracle.  Tolerance: the prompt bound times 1.6 -- a prompt of 500 tokens has
    ten times the bf16 roundings of the 41-token prompts above to flip (measured here: up to 4.7e-3, the same to three
    digits on both paths); every mutation of the sensitivity test stays five times above it."""
    import dataclasses

    tol = 1.6 * PROMPT_TOL

    cfg = dataclasses.replace(CASES[case], max_tokens=640)
    w = llama.conditioned_weights(cfg, SEED)
    key = (case, "long", prompt_len)
    if key not in _ORACLE:
        ora = OracleLlama(cfg, w)
        prompt = tokens(prompt_len, cfg.vocab, seed=6)
        ora.prefill(prompt, bf16_gemm=True)
        first = ora.logits.copy()
        toks = tokens(30, cfg.vocab, seed=8)
        out = []
        for t in toks:
            ora.step(t)
            out.append(ora.logits.copy())
        _ORACLE[key] = (prompt, first, toks, out)
    prompt, first, toks, want = _ORACLE[key]
    hip.set_option("llama.attn_wide", wide)
    try:
        model = llama.LlamaModel(hip, cfg, weights=w)
        model.prefill(prompt)
        worst = logit_err(model.logits(), first)
        assert worst <= tol, (case, "prompt", worst)
        for i, t in enumerate(toks):
            model.decode(t, 1)
            err = logit_err(model.logits(), want[i])
            worst = max(worst, err)
            assert err <= tol, (case, wide, i, err)
        print(f"{case} prompt {prompt_len} wide={wide}: worst logit error {worst:.2e}")
        model.free()
    finally:
        hip.set_option("llama.attn_wide", 1)


_HEAD_DIMS = {
    # eight heads of 64 (prompt attention and rotary pairs at the smaller head), four cached
    "hd64": llama.Config(n_layer=2, hidden=512, ffn=768, n_head=8, n_kv_head=4, head_dim=64, vocab=512, max_tokens=96, page_tokens=16),
    # two heads of 256: the prompt has no matrix-core attention at this size and takes the decode kernel, one query
    # row per prompt token
    "hd256": llama.Config(n_layer=2, hidden=512, ffn=768, n_head=2, n_kv_head=1, head_dim=256, vocab=512, max_tokens=96, page_tokens=16),
}


@pytest.mark.parametrize("splits", [0, 1])
@pytest.mark.parametrize("name", list(_HEAD_DIMS))
def test_other_head_sizes_prompt_then_decode(hip, name, splits):
    """head_dim 64 and 256 through the prompt path and the decode path (the cases above are all 128): a prompt of 70
    tokens -- two splits of the attention where the prompt takes the decode kernel -- and 24 steps, with the split count
    the library chooses and with one."""
    cfg = _HEAD_DIMS[name]
    weights = llama.conditioned_weights(cfg, SEED)
    ora = OracleLlama(cfg, weights)
    prompt = tokens(70, cfg.vocab, seed=2)
    ora.prefill(prompt, bf16_gemm=True)
    first = ora.logits.copy()
    toks = tokens(24, cfg.vocab, seed=4)
    hip.set_option("attn.splits", splits)
    try:
        model = llama.LlamaModel(hip, cfg, weights=weights)
        model.prefill(prompt)
        worst = logit_err(model.logits(), first)
        assert worst <= PROMPT_TOL, (name, "prompt", worst)
        for i, t in enumerate(toks):
            ora.step(t)
            model.decode(t, 1)
            err = logit_err(model.logits(), ora.logits)
            worst = max(worst, err)
            assert err <= PROMPT_TOL, (name, splits, i, err)
        print(f"{name} splits={splits}: worst logit error {worst:.2e}")
        model.free()
    finally:
        hip.set_option("attn.splits", 0)
