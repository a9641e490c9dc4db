"""Writes tests/golden/cfg5_llama7b_512_128.npz: the CPU oracle's answer for the 7B-shaped decoder at its stated length.

    python tests/golden/make_cfg5_golden.py [--state /tmp/cfg5_state.npz]

Model: llama.Config() (32 distinct layers, hidden 4096, FFN 11008, 32 heads x 128, vocabulary 32000, Q4_K layers,
Q6_K head), llama.random_weights(cfg, seed=11).  Input: the 512 ids np.random.default_rng(11).integers(0, 32000, 512).
The oracle (oracle/llama_oracle.py: C kernels, fp64 accumulation, one token at a time) runs the prompt with the
activations of every projection rounded to bf16 -- what the library's prompt GEMMs are fed -- and then 128 greedy
steps in fp32.  Stored: the prompt, the greedy token of every step, and for the prompt's last token and the decode
steps 0, 1, 63 and 127 every eighth logit together with the vector's largest magnitude, its arg max and its top-two
margin (the error metric is relative to the largest magnitude).

The run takes about 55 minutes on 8 cores (640 tokens x 3.75 GB of blocks); it keeps its state in --state every 32
tokens and resumes from there.
"""
from __future__ import annotations

import argparse
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle.llama_oracle import OracleLlama  # noqa: E402
from skainet_amd import llama  # noqa: E402

SEED, PROMPT_LEN, STEPS, STRIDE = 11, 512, 128, 8
KEEP = (0, 1, 63, 127)
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cfg5_llama7b_512_128.npz")


def summary(logits):
    s = np.sort(logits)
    return (logits[::STRIDE].astype(np.float32), np.float32(np.abs(logits).max()), np.int32(np.argmax(logits)),
            np.float32(s[-1] - s[-2]))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--state", default="/tmp/cfg5_state.npz")
    args = ap.parse_args()
    cfg = llama.Config(max_tokens=1024)
    t0 = time.time()
    w = llama.random_weights(cfg, seed=SEED)
    print(f"weights built in {time.time() - t0:.0f} s", flush=True)
    prompt = np.random.default_rng(SEED).integers(0, cfg.vocab, size=PROMPT_LEN).astype(np.int32)
    ora = OracleLlama(cfg, w)
    tokens, kept = [], {}
    if os.path.exists(args.state):
        st = np.load(args.state)
        ora.k[:, : int(st["pos"])] = st["k"]
        ora.v[:, : int(st["pos"])] = st["v"]
        ora.pos = int(st["pos"])
        tokens = st["tokens"].tolist()
        kept = {key[5:]: st[key] for key in st.files if key.startswith("kept_")}
        print(f"resumed at position {ora.pos}", flush=True)

    def save_state():
        np.savez(args.state + ".tmp.npz", k=ora.k[:, : ora.pos], v=ora.v[:, : ora.pos], pos=ora.pos,
                 tokens=np.array(tokens, np.int32), **{f"kept_{k}": v for k, v in kept.items()})
        os.replace(args.state + ".tmp.npz", args.state)

    def keep(tag, logits):
        for name, val in zip(("sample", "absmax", "argmax", "margin"), summary(logits)):
            kept[f"{tag}_{name}"] = val

    t0 = time.time()
    while ora.pos < PROMPT_LEN:
        last = ora.pos == PROMPT_LEN - 1
        nxt = ora.step(int(prompt[ora.pos]), bf16_gemm=True, want_logits=last)
        if last:
            keep("prefill", ora.logits)
            tokens = [int(nxt)]  # tokens[0] = the prompt's greedy continuation, fed to decode step 0
        if ora.pos % 32 == 0:
            save_state()
            print(f"prompt {ora.pos}/{PROMPT_LEN}  {time.time() - t0:.0f} s", flush=True)
    while ora.pos < PROMPT_LEN + STEPS:
        i = ora.pos - PROMPT_LEN
        tok = ora.step(tokens[i])
        tokens.append(int(tok))
        if i in KEEP:
            keep(f"step{i}", ora.logits)
        if ora.pos % 32 == 0 or i == STEPS - 1:
            save_state()
            print(f"decode {i + 1}/{STEPS}  {time.time() - t0:.0f} s", flush=True)
    np.savez_compressed(OUT, seed=np.int32(SEED), stride=np.int32(STRIDE), prompt=prompt,
                        first=np.int32(tokens[0]), tokens=np.array(tokens[1:], np.int32), **kept)
    print(f"wrote {OUT} ({os.path.getsize(OUT)} bytes)")


if __name__ == "__main__":
    main()
