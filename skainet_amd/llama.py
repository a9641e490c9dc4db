"""Host side of the Llama-style decoder: seeded random-init GGUF-block weights, upload, prefill and greedy decode.

The module graph is the reference's nested Module.forward composition (core/src/commonMain/kotlin/sk/ai/net/nn/
Module.kt:6-16, nn/topology/MLP.kt:13-19) instantiated for a Llama block stack; every Linear
(nn/Linear.kt:43-49, y = x . W^T, no bias here) holds a quantized [out, in] weight on the device.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field

import numpy as np

from . import runtime, synth
from .runtime import Q4_K, Q6_K, LlamaConfig, LlamaLayer, LlamaWeights


@dataclass
class Config:
    n_layer: int = 32
    hidden: int = 4096
    ffn: int = 11008
    n_head: int = 32
    head_dim: int = 128
    vocab: int = 32000
    max_tokens: int = 1024
    page_tokens: int = 256
    rope_base: float = 10000.0
    rms_eps: float = 1e-5
    n_kv_head: int = 0      # heads of wk / wv and of the cache (grouped-query attention); 0 = n_head
    type_attn: int = Q4_K   # wq, wk, wv, wo unless overridden below
    type_ffn: int = Q4_K    # w_gate, w_up, w_down unless overridden below
    type_embd: int = Q4_K
    type_head: int = Q6_K
    # Per-matrix overrides, the way mixed quantizations give some matrices more bits: keys are a matrix name
    # ("wv", "w_down", ...) for every layer or "l<layer>.<name>" for one layer.
    matrix_types: dict = field(default_factory=dict)

    @property
    def kv_heads(self) -> int:
        return self.n_kv_head or self.n_head

    def matrix_type(self, layer: int, name: str) -> int:
        default = self.type_attn if name in ("wq", "wk", "wv", "wo") else self.type_ffn
        return self.matrix_types.get(f"l{layer}.{name}", self.matrix_types.get(name, default))


LLAMA_7B = Config()


def random_weights(cfg: Config, seed: int):
    """Host copy of a seeded random-init model: dict name -> (ggml type or None for fp32, ndarray)."""
    h, f, v = cfg.hidden, cfg.ffn, cfg.vocab
    w = {}
    rng = np.random.default_rng(seed)
    w["tok_embd"] = (cfg.type_embd, synth.weight(cfg.type_embd, v, h, seed + 1))
    w["out_head"] = (cfg.type_head, synth.weight(cfg.type_head, v, h, seed + 2))
    w["out_norm"] = (None, (1.0 + 0.1 * rng.standard_normal(h)).astype(np.float32))
    for l in range(cfg.n_layer):
        s = seed + 100 * (l + 1)
        kvd = cfg.kv_heads * cfg.head_dim
        for i, name in enumerate(("wq", "wk", "wv", "wo")):
            t = cfg.matrix_type(l, name)
            w[f"l{l}.{name}"] = (t, synth.weight(t, kvd if name in ("wk", "wv") else h, h, s + i))
        for i, (name, rows, cols) in enumerate((("w_gate", f, h), ("w_up", f, h), ("w_down", h, f))):
            t = cfg.matrix_type(l, name)
            w[f"l{l}.{name}"] = (t, synth.weight(t, rows, cols, s + 10 + i))
        w[f"l{l}.attn_norm"] = (None, (1.0 + 0.1 * rng.standard_normal(h)).astype(np.float32))
        w[f"l{l}.ffn_norm"] = (None, (1.0 + 0.1 * rng.standard_normal(h)).astype(np.float32))
    return w


# Gains of the conditioned model: queries and keys of rms about 1 give attention scores of order one (larger ones make
# the logits hang on single fp16 roundings of cached keys), the attention branch (values 1, output projection 1.5)
# outweighs the feed-forward branch (gate / up 1, down 1 on a SwiGLU of rms about 0.4), and the residual stream stays
# of order one through the stack.
_GAINS = {"wq": 1.0, "wk": 1.0, "wv": 1.0, "wo": 1.5, "w_gate": 1.0, "w_up": 1.0, "w_down": 1.0}


def conditioned_weights(cfg: Config, seed: int, gains=None):
    """Like random_weights, with every matrix drawn by synth.conditioned_weight: zero-centred values and a power-of-two
    scale per matrix, so that the logits depend on positions, on the cache and on the attention (the benchmark's
    Q4_K draws have a mean that buries those under the feed-forward output).  The model for decoder parity tests."""
    h, f, v = cfg.hidden, cfg.ffn, cfg.vocab
    gains = {**_GAINS, **(gains or {})}
    w = {}
    rng = np.random.default_rng(seed)
    w["tok_embd"] = (cfg.type_embd, synth.conditioned_weight(cfg.type_embd, v, h, seed + 1, gain=np.sqrt(h)))
    w["out_head"] = (cfg.type_head, synth.conditioned_weight(cfg.type_head, v, h, seed + 2, gain=1.0))
    w["out_norm"] = (None, (1.0 + 0.1 * rng.standard_normal(h)).astype(np.float32))
    kvd = cfg.kv_heads * cfg.head_dim
    shapes = {"wq": (h, h), "wk": (kvd, h), "wv": (kvd, h), "wo": (h, h), "w_gate": (f, h), "w_up": (f, h), "w_down": (h, f)}
    for l in range(cfg.n_layer):
        s = seed + 100 * (l + 1)
        for i, (name, (rows, cols)) in enumerate(shapes.items()):
            t = cfg.matrix_type(l, name)
            w[f"l{l}.{name}"] = (t, synth.conditioned_weight(t, rows, cols, s + i, gain=gains[name]))
        w[f"l{l}.attn_norm"] = (None, (1.0 + 0.1 * rng.standard_normal(h)).astype(np.float32))
        w[f"l{l}.ffn_norm"] = (None, (1.0 + 0.1 * rng.standard_normal(h)).astype(np.float32))
    return w


class LlamaModel:
    """Device-resident model: owns the uploaded weights and the skn_llama handle."""

    def __init__(self, ctx: runtime.Context, cfg: Config, weights=None, seed: int = 0, share_layers: bool = False):
        """share_layers=True uploads one layer's weights and points every layer at them (shape-faithful timing
        of a model larger than one wants to generate on the host; never used for parity)."""
        self.ctx, self.cfg = ctx, cfg
        self.bufs = {}
        if weights is None:
            gen_cfg = cfg if not share_layers else Config(**{**cfg.__dict__, "n_layer": 1})
            weights = random_weights(gen_cfg, seed)
        self.host_weights = weights if not share_layers else None
        self.head_type = weights["out_head"][0]
        uploaded = {}  # an array that appears under two names (a head tied to the embedding) is uploaded once
        for name, (_, arr) in weights.items():
            if id(arr) not in uploaded:
                uploaded[id(arr)] = ctx.to_device(arr)
            self.bufs[name] = uploaded[id(arr)]
        layers = (LlamaLayer * cfg.n_layer)()
        for l in range(cfg.n_layer):
            src = 0 if share_layers else l
            L = layers[l]
            for f in ("wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down", "attn_norm", "ffn_norm"):
                setattr(L, f, self.bufs[f"l{src}.{f}"].ptr)
            for f, tf in (("wq", "type_q"), ("wk", "type_k"), ("wv", "type_v"), ("wo", "type_o"), ("w_gate", "type_gate"),
                          ("w_up", "type_up"), ("w_down", "type_down")):
                setattr(L, tf, weights[f"l{src}.{f}"][0])  # the type each matrix was built with
        self._layers = layers
        wts = LlamaWeights(self.bufs["tok_embd"].ptr, self.bufs["out_norm"].ptr, self.bufs["out_head"].ptr,
                           weights["tok_embd"][0], weights["out_head"][0], layers)
        c = LlamaConfig(cfg.n_layer, cfg.hidden, cfg.ffn, cfg.n_head, cfg.head_dim, cfg.vocab, cfg.max_tokens,
                        cfg.page_tokens, cfg.rope_base, cfg.rms_eps, cfg.n_kv_head)
        h = C.c_void_p()
        ctx._check(ctx.lib.skn_llama_create(ctx.handle, C.byref(c), C.byref(wts), C.byref(h)))
        self.handle = h.value

    def reset(self):
        self.ctx._check(self.ctx.lib.skn_llama_reset(self.ctx.handle, self.handle))

    def prefill(self, tokens):
        arr = (C.c_int32 * len(tokens))(*[int(t) for t in tokens])
        nxt = C.c_int32()
        self.ctx._check(self.ctx.lib.skn_llama_prefill(self.ctx.handle, self.handle, arr, len(tokens), C.byref(nxt)))
        return nxt.value

    def decode(self, first_token, n_steps):
        out = (C.c_int32 * max(n_steps, 1))()
        self.ctx._check(self.ctx.lib.skn_llama_decode(self.ctx.handle, self.handle, int(first_token), n_steps, out))
        return list(out[:n_steps])

    def logits(self):
        p = C.c_void_p()
        self.ctx._check(self.ctx.lib.skn_llama_logits(self.ctx.handle, self.handle, C.byref(p)))
        out = np.empty(self.cfg.vocab, dtype=np.float32)
        self.ctx._check(self.ctx.lib.skn_download(self.ctx.handle, out.ctypes.data, p.value, out.nbytes))
        return out

    def free(self):
        if self.handle:
            self.ctx.lib.skn_llama_free(self.ctx.handle, self.handle)
            self.handle = None
        for b in {id(b): b for b in self.bufs.values()}.values():
            b.free()
        self.bufs = {}

    def weight_bytes_per_token(self):
        """Bytes of weights one decode step streams (embedding row excluded): the HBM floor of a token."""
        c = self.cfg

        def rb(t, n, k):
            be, bb = synth.BLOCK[t]
            return n * (k // be) * bb

        total = rb(self.head_type, c.vocab, c.hidden)
        for l in range(c.n_layer):
            total += sum(rb(c.matrix_type(l, nm), c.hidden, c.hidden) for nm in ("wq", "wo"))
            total += sum(rb(c.matrix_type(l, nm), c.kv_heads * c.head_dim, c.hidden) for nm in ("wk", "wv"))
            total += sum(rb(c.matrix_type(l, nm), c.ffn, c.hidden) for nm in ("w_gate", "w_up"))
            total += rb(c.matrix_type(l, "w_down"), c.hidden, c.ffn)
        return total


# ---- a model out of a GGUF file ---------------------------------------------------------------------------------
# Tensor and metadata names are those of llama.cpp's GGUF files for the "llama" architecture, the files the
# reference's reader is written for (gguf/src/commonMain/kotlin/sk/ai/net/gguf/GGUFReader.kt:82-139 reads the key /
# value fields, :332-401 the tensors).  Their q and k projections are stored for the rotary embedding of adjacent
# pairs (2i, 2i + 1), which is the convention of this decoder.
_GGUF_LAYER_TENSORS = {"wq": "attn_q", "wk": "attn_k", "wv": "attn_v", "wo": "attn_output", "w_gate": "ffn_gate",
                       "w_up": "ffn_up", "w_down": "ffn_down"}


def config_from_gguf(reader, max_tokens=None, page_tokens=256) -> Config:
    """The decoder's shape from the metadata of an opened GGUFReader (ValueError when a field is missing or the
    file describes something this decoder does not compute)."""
    f = reader.fields
    arch = f.get("general.architecture")
    if arch != "llama":
        raise ValueError(f"general.architecture is {arch!r}: only 'llama' files are decoded")

    def need(key):
        if f"{arch}.{key}" not in f:
            raise ValueError(f"GGUF metadata lacks {arch}.{key}")
        return f[f"{arch}.{key}"]

    hidden, n_head = int(need("embedding_length")), int(need("attention.head_count"))
    head_dim = int(f.get(f"{arch}.attention.key_length", hidden // n_head))
    rope_dims = int(f.get(f"{arch}.rope.dimension_count", head_dim))
    if rope_dims != head_dim:
        raise ValueError(f"partial rotary embedding ({rope_dims} of {head_dim} dimensions) is not supported")
    embd = reader.tensor("token_embd.weight")
    n_kv = int(f.get(f"{arch}.attention.head_count_kv", n_head))
    return Config(
        n_layer=int(need("block_count")), hidden=hidden, ffn=int(need("feed_forward_length")), n_head=n_head,
        head_dim=head_dim, vocab=int(embd.shape[0]),
        max_tokens=int(max_tokens or f.get(f"{arch}.context_length", 2048)), page_tokens=page_tokens,
        rope_base=float(f.get(f"{arch}.rope.freq_base", 10000.0)),
        rms_eps=float(f.get(f"{arch}.attention.layer_norm_rms_epsilon", 1e-5)),
        n_kv_head=0 if n_kv == n_head else n_kv, type_embd=embd.tensor_type)


def weights_from_gguf(reader, cfg: Config):
    """name -> (ggml type or None for fp32 vectors, array) in the form LlamaModel takes; the arrays are views of the
    mapped file.  A file without output.weight shares the embedding table with the head."""
    names = {t.name for t in reader.tensors}

    def matrix(name, rows, cols):
        t = reader.tensor(name)
        if t.shape != (rows, cols):
            raise ValueError(f"{name} is {t.shape}, expected {(rows, cols)}")
        return (t.tensor_type, t.data if t.data.dtype == np.uint8 else np.ascontiguousarray(t.data).view(np.uint8).reshape(-1))

    def vector(name, n):
        t = reader.tensor(name)
        if t.shape != (n,):
            raise ValueError(f"{name} is {t.shape}, expected {(n,)}")
        return (None, np.ascontiguousarray(t.data, dtype=np.float32))

    h, kvd = cfg.hidden, cfg.kv_heads * cfg.head_dim
    w = {"tok_embd": matrix("token_embd.weight", cfg.vocab, h), "out_norm": vector("output_norm.weight", h)}
    w["out_head"] = matrix("output.weight", cfg.vocab, h) if "output.weight" in names else w["tok_embd"]
    shapes = {"wq": (h, h), "wk": (kvd, h), "wv": (kvd, h), "wo": (h, h), "w_gate": (cfg.ffn, h), "w_up": (cfg.ffn, h),
              "w_down": (h, cfg.ffn)}
    for l in range(cfg.n_layer):
        for ours, theirs in _GGUF_LAYER_TENSORS.items():
            w[f"l{l}.{ours}"] = matrix(f"blk.{l}.{theirs}.weight", *shapes[ours])
        w[f"l{l}.attn_norm"] = vector(f"blk.{l}.attn_norm.weight", h)
        w[f"l{l}.ffn_norm"] = vector(f"blk.{l}.ffn_norm.weight", h)
    return w


def model_from_gguf(ctx: runtime.Context, path: str, max_tokens=None, page_tokens=256) -> LlamaModel:
    """Opens a llama-architecture GGUF file, uploads its tensors as they are and returns the decoder over them."""
    from . import gguf

    reader = gguf.GGUFReader(path)
    try:
        cfg = config_from_gguf(reader, max_tokens, page_tokens)
        w = weights_from_gguf(reader, cfg)
        cfg.type_head = w["out_head"][0]
        model = LlamaModel(ctx, cfg, weights=w)
        model.host_weights = None  # (views of the mapped file: not kept)
        del w
        return model
    finally:
        reader.close()


def write_gguf_model(path, cfg: Config, weights):
    """The inverse, for tests and for handing a synthetic model to other GGUF consumers."""
    from . import gguf

    fields = {"general.architecture": "llama", "llama.block_count": cfg.n_layer, "llama.embedding_length": cfg.hidden,
              "llama.feed_forward_length": cfg.ffn, "llama.attention.head_count": cfg.n_head,
              "llama.attention.head_count_kv": cfg.kv_heads, "llama.context_length": cfg.max_tokens,
              "llama.rope.freq_base": float(cfg.rope_base), "llama.attention.layer_norm_rms_epsilon": float(cfg.rms_eps)}
    h, kvd = cfg.hidden, cfg.kv_heads * cfg.head_dim
    shapes = {"wq": (h, h), "wk": (kvd, h), "wv": (kvd, h), "wo": (h, h), "w_gate": (cfg.ffn, h), "w_up": (cfg.ffn, h),
              "w_down": (h, cfg.ffn)}
    tensors = [("token_embd.weight", weights["tok_embd"][0], (cfg.vocab, h), weights["tok_embd"][1]),
               ("output_norm.weight", 0, (h,), weights["out_norm"][1]),
               ("output.weight", weights["out_head"][0], (cfg.vocab, h), weights["out_head"][1])]
    for l in range(cfg.n_layer):
        for ours, theirs in _GGUF_LAYER_TENSORS.items():
            t, arr = weights[f"l{l}.{ours}"]
            tensors.append((f"blk.{l}.{theirs}.weight", t, shapes[ours], arr))
        tensors.append((f"blk.{l}.attn_norm.weight", 0, (h,), weights[f"l{l}.attn_norm"][1]))
        tensors.append((f"blk.{l}.ffn_norm.weight", 0, (h,), weights[f"l{l}.ffn_norm"][1]))
    gguf.write_gguf(path, fields, tensors)

