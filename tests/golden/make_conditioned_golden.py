"""Writes tests/golden/conditioned_4layer_512_128.npz: the CPU oracle's answer for a decoder of the 7B model's width at
the benchmark's length, on weights whose logits depend on positions and attention.

    python tests/golden/make_conditioned_golden.py

Model: llama.Config(n_layer=4, max_tokens=1024) -- four distinct layers of hidden 4096, FFN 11008, 32 heads x 128,
vocabulary 32000, Q4_K layers and embedding, Q6_K head -- with llama.conditioned_weights(cfg, seed=17) (zero-centred
values, a power-of-two scale per matrix; the benchmark's own draws bury the attention under the feed-forward
output).  Input: 512 ids np.random.default_rng(17).integers(0, 32000, 512).  The oracle (oracle/llama_oracle.py) runs
the prompt with the activations of every projection rounded to bf16, as the library's prompt GEMMs are fed, then 128
greedy steps in fp32 (context 513 to 640: the 2 -> 3 page boundary of 256-token pages at the first step).  Stored: the
prompt, the greedy token of every step, every eighth logit of the prompt's last row and of steps 0, 1, 31, 63, 95, 127
with each vector's largest magnitude, arg max and top-two margin; and, from the first 40 tokens of the same prompt
run in fp32, how far each mutation of oracle/llama_oracle.py moves the logits (smallest and median over the steps
from the third on, as max |difference| / max |logit|).

About 10 minutes on 8 cores.
"""
from __future__ import annotations

import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle.llama_oracle import MUTATIONS, OracleLlama  # noqa: E402
from skainet_amd import llama  # noqa: E402

SEED, PROMPT_LEN, STEPS, STRIDE, N_LAYER = 17, 512, 128, 8, 4
KEEP = (0, 1, 31, 63, 95, 127)
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "conditioned_4layer_512_128.npz")


def config():
    return llama.Config(n_layer=N_LAYER, max_tokens=1024)


def summary(logits):
    s = np.sort(logits)
    return (logits[::STRIDE].astype(np.float32), np.float32(np.abs(logits).max()), np.int32(np.argmax(logits)),
            np.float32(s[-1] - s[-2]))


def main():
    cfg = config()
    t0 = time.time()
    w = llama.conditioned_weights(cfg, seed=SEED)
    print(f"weights built in {time.time() - t0:.0f} s", flush=True)
    prompt = np.random.default_rng(SEED).integers(0, cfg.vocab, size=PROMPT_LEN).astype(np.int32)
    kept = {}

    def keep(tag, logits):
        for name, val in zip(("sample", "absmax", "argmax", "margin"), summary(logits)):
            kept[f"{tag}_{name}"] = val

    # sensitivity of this model: 40 tokens, every mutation against the unmodified run
    def short_run(mutation):
        o = OracleLlama(cfg, w, mutation)
        out = []
        for t in prompt[:40]:
            o.step(int(t))
            out.append(o.logits.copy())
        return out

    base = short_run(None)
    for m in MUTATIONS:
        if m == "kv_head_mod":
            continue  # (as many cached heads as query heads here)
        e = np.array([np.abs(a - b).max() / np.abs(b).max() for a, b in zip(short_run(m), base)])[2:]
        kept[f"mutation_{m}_min"], kept[f"mutation_{m}_median"] = np.float32(e.min()), np.float32(np.median(e))
        print(f"mutation {m}: min {e.min():.3f} median {np.median(e):.3f}  {time.time() - t0:.0f} s", flush=True)

    ora = OracleLlama(cfg, w)
    tokens = []
    while ora.pos < PROMPT_LEN:
        last = ora.pos == PROMPT_LEN - 1
        nxt = ora.step(int(prompt[ora.pos]), bf16_gemm=True, want_logits=last)
        if last:
            keep("prefill", ora.logits)
            tokens = [int(nxt)]  # tokens[0] = the prompt's greedy continuation, fed to decode step 0
        if ora.pos % 64 == 0:
            print(f"prompt {ora.pos}/{PROMPT_LEN}  {time.time() - t0:.0f} s", flush=True)
    for i in range(STEPS):
        tok = ora.step(tokens[i])
        tokens.append(int(tok))
        if i in KEEP:
            keep(f"step{i}", ora.logits)
    print(f"decode done  {time.time() - t0:.0f} s; distinct greedy tokens: {len(set(tokens))}", flush=True)
    np.savez_compressed(OUT, seed=np.int32(SEED), stride=np.int32(STRIDE), n_layer=np.int32(N_LAYER), prompt=prompt,
                        first=np.int32(tokens[0]), tokens=np.array(tokens[1:], np.int32), **kept)
    print(f"wrote {OUT} ({os.path.getsize(OUT)} bytes)")


if __name__ == "__main__":
    main()
