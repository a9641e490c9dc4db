"""CPU oracle of the Llama-style decoder (test infrastructure only): the same module graph evaluated with the C
oracle's kernels (fp64 accumulation), token by token.  Prompt tokens can be run either exactly like decode steps
(`bf16_gemm=False`) or with the activations of every projection rounded to bf16 first (`bf16_gemm=True`), which is
what the batched prompt path of the library feeds its GEMMs with.

`mutation` swaps in one deliberately wrong piece (tests use it to show that a model's logits react to that piece, i.e.
that a parity test on that model could catch such a mistake): "no_rope" (rotary embedding skipped), "pos_plus_one"
(the query rotated for the next position, the key for its own: relative positions off by one -- shifting queries and
keys alike would change nothing, the rotary embedding being relative), "ctx_minus_one" (the attention leaves out the newest token), "last_only" (the attention
sees the newest token only), "kv_head_mod" (query head i reads cached head i % kv heads instead of i // group)."""
from __future__ import annotations

import numpy as np

from . import oracle_c, oracle_np


MUTATIONS = ("no_rope", "pos_plus_one", "ctx_minus_one", "last_only", "kv_head_mod")


class OracleLlama:
    def __init__(self, cfg, weights, mutation=None):
        assert mutation is None or mutation in MUTATIONS, mutation
        self.cfg, self.w, self.mutation = cfg, weights, mutation
        c = cfg
        self.kvh = getattr(c, "n_kv_head", 0) or c.n_head  # grouped-query attention: heads of k / v
        self.k = np.zeros((c.n_layer, c.max_tokens, self.kvh, c.head_dim), dtype=np.uint16)
        self.v = np.zeros_like(self.k)
        self.pos = 0
        self.logits = None

    def _lin(self, name, n, k, x, bf16):
        t, raw = self.w[name]
        if bf16:
            x = oracle_np.bf16_to_f32(oracle_np.f32_to_bf16(x))
        return oracle_c.matvec_q(t, raw, n, k, x)

    def step(self, token, bf16_gemm=False, want_logits=True):
        c = self.cfg
        h, f = c.hidden, c.ffn
        t, raw = self.w["tok_embd"]
        be, bb = oracle_c.type_sizes(t)
        rb = h // be * bb
        x = oracle_c.dequant(t, raw[token * rb:(token + 1) * rb], h)
        pos, mut = self.pos, self.mutation
        for l in range(c.n_layer):
            xn = oracle_c.rmsnorm(x, self.w[f"l{l}.attn_norm"][1], c.rms_eps)
            q = self._lin(f"l{l}.wq", h, h, xn, bf16_gemm).reshape(c.n_head, c.head_dim)
            kvd = self.kvh * c.head_dim
            k = self._lin(f"l{l}.wk", kvd, h, xn, bf16_gemm).reshape(self.kvh, c.head_dim)
            v = self._lin(f"l{l}.wv", kvd, h, xn, bf16_gemm).reshape(self.kvh, c.head_dim)
            if mut != "no_rope":
                q = oracle_c.rope(q, pos + 1 if mut == "pos_plus_one" else pos, c.rope_base)
                k = oracle_c.rope(k, pos, c.rope_base)
            self.k[l, pos] = oracle_c.f2h(k)
            self.v[l, pos] = oracle_c.f2h(v)
            # query head i reads cached head i // (n_head / kv heads)
            rep = c.n_head // self.kvh
            lo, hi = 0, pos + 1
            if mut == "ctx_minus_one" and pos > 0:
                hi = pos
            if mut == "last_only":
                lo = pos
            kc, vc = self.k[l][None, lo:hi], self.v[l][None, lo:hi]
            if mut == "kv_head_mod":
                heads = np.arange(c.n_head) % self.kvh
                kc, vc = kc[:, :, heads], vc[:, :, heads]
            else:
                kc, vc = np.repeat(kc, rep, axis=2), np.repeat(vc, rep, axis=2)
            att = oracle_c.attn_decode(q[None], kc, vc, [hi - lo], 1.0 / np.sqrt(c.head_dim))[0].reshape(h)
            x = x + self._lin(f"l{l}.wo", h, h, att, bf16_gemm)
            xn = oracle_c.rmsnorm(x, self.w[f"l{l}.ffn_norm"][1], c.rms_eps)
            g = self._lin(f"l{l}.w_gate", f, h, xn, bf16_gemm)
            u = self._lin(f"l{l}.w_up", f, h, xn, bf16_gemm)
            x = x + self._lin(f"l{l}.w_down", h, f, oracle_c.swiglu(g, u), bf16_gemm)
        self.pos += 1
        if want_logits:
            xn = oracle_c.rmsnorm(x, self.w["out_norm"][1], c.rms_eps)
            self.logits = self._lin("out_head", c.vocab, h, xn, False)
            return oracle_c.argmax(self.logits)
        return None

    def prefill(self, tokens, bf16_gemm=True):
        nxt = None
        for i, t in enumerate(tokens):
            nxt = self.step(int(t), bf16_gemm=bf16_gemm, want_logits=(i == len(tokens) - 1))
        return nxt

    def decode(self, first_token, n_steps):
        out, tok = [], int(first_token)
        for _ in range(n_steps):
            tok = self.step(tok)
            out.append(tok)
        return out
