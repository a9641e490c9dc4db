"""NumPy oracle for the quantized-inference hot path.  TEST INFRASTRUCTURE ONLY.

A second restatement, written independently of ``oracle/oracle.c`` and in a different
form: whole-tensor vectorised bit manipulation, values formed in float64 from the closed
form and rounded ONCE to float32.  Because every intermediate product of the ggml block
formulas is exactly representable (f16 scale: 11 bits, 6/8-bit sub-scale, 4/6-bit quant),
"fp64 closed form rounded once" and "the fp32 instruction sequence" must agree bit for bit;
the tests assert that the two oracles do.

Followed sources:
  * block sizes / type ids: reference gguf/src/commonMain/kotlin/sk/ai/net/gguf/Constants.kt:14-52,58-90
  * byte-row shape rule:    reference gguf/src/commonMain/kotlin/sk/ai/net/gguf/Quants.kt:10-20
  * dense matmul semantics: reference core/src/commonMain/kotlin/sk/ai/net/impl/DoublesTensor.kt:255-279
  * Linear:                 reference core/src/commonMain/kotlin/sk/ai/net/nn/Linear.kt:43-49
  * bit packing of Q8_0 / Q4_K / Q6_K: absent from the reference (Quants.kt:8 TODO); the public
    ggml block definitions the reference cites as its origin (Quants.kt:4-5).

Nothing in the product path may import this module; only tests, the smoke check and the
bench's cpu_baseline leg do.
"""
from __future__ import annotations

import numpy as np

Q8_0, Q4_K, Q6_K = 8, 12, 14
F32, F16, BF16 = 0, 1, 30
Q4_0, Q4_1, Q5_0, Q5_1, Q2_K, Q5_K = 2, 3, 6, 7, 10, 13
Q3_K, Q8_K, IQ4_NL, IQ4_XS = 11, 15, 20, 23
TQ1_0, TQ2_0 = 34, 35

# Constants.kt:58-90 restricted to the types this library computes with: type -> (block elems, block bytes)
QUANT_SIZES = {
    F32: (1, 4),
    F16: (1, 2),
    BF16: (1, 2),
    Q4_0: (32, 2 + 16),
    Q4_1: (32, 2 + 2 + 16),
    Q5_0: (32, 2 + 4 + 16),
    Q5_1: (32, 2 + 2 + 4 + 16),
    Q8_0: (32, 2 + 32),
    Q2_K: (256, 2 + 2 + 256 // 16 + 256 // 4),
    Q4_K: (256, 2 + 2 + 256 // 2 + 12),
    Q5_K: (256, 2 + 2 + 256 // 2 + 256 // 8 + 12),
    Q6_K: (256, 2 + 256 // 2 + 256 // 4 + 256 // 16),
    Q3_K: (256, 2 + 256 // 4 + 256 // 8 + 12),
    Q8_K: (256, 4 + 256 + 256 // 8),
    IQ4_NL: (32, 2 + 16),
    IQ4_XS: (256, 2 + 2 + 256 // 2 + 256 // 64),
    TQ1_0: (256, 2 + 4 * 13),
    TQ2_0: (256, 2 + 64),
}
TYPE_NAMES = {Q8_0: "Q8_0", Q4_K: "Q4_K", Q6_K: "Q6_K", F32: "F32", F16: "F16", BF16: "BF16", Q4_0: "Q4_0",
              Q4_1: "Q4_1", Q5_0: "Q5_0", Q5_1: "Q5_1", Q2_K: "Q2_K", Q5_K: "Q5_K", Q3_K: "Q3_K", Q8_K: "Q8_K",
              IQ4_NL: "IQ4_NL", IQ4_XS: "IQ4_XS", TQ1_0: "TQ1_0", TQ2_0: "TQ2_0"}


def quant_shape_to_byte_shape(shape, qtype):
    """Quants.kt:10-20, same message on a bad row size."""
    block, tsize = QUANT_SIZES[qtype]
    if shape[-1] % block != 0:
        raise ValueError(
            f"Quantized tensor row size ({shape[-1]}) is not a multiple of {TYPE_NAMES[qtype]} block size ({block})"
        )
    return tuple(shape[:-1]) + (shape[-1] // block * tsize,)


def _blocks(raw, qtype):
    raw = np.ascontiguousarray(np.frombuffer(raw, dtype=np.uint8) if not isinstance(raw, np.ndarray) else raw)
    raw = raw.reshape(-1).view(np.uint8)
    bb = QUANT_SIZES[qtype][1]
    if raw.size % bb:
        raise ValueError("byte count is not a whole number of blocks")
    return raw.reshape(-1, bb)


def _f16(col_bytes):
    """two uint8 columns -> float64 values of the little-endian binary16 they hold (numpy's converter)."""
    return np.ascontiguousarray(col_bytes).view("<f2").astype(np.float64).reshape(-1)


def dequant_q8_0(raw):
    b = _blocks(raw, Q8_0)
    d = _f16(b[:, 0:2])
    q = b[:, 2:34].view(np.int8).astype(np.float64)
    return (d[:, None] * q).astype(np.float32).reshape(-1)


def q4k_scales_mins(scales12):
    """[nb,12] uint8 -> (sc [nb,8], m [nb,8]) 6-bit values, written with whole-array masks."""
    s = scales12.astype(np.uint16)
    sc = np.empty(s.shape[:-1] + (8,), dtype=np.uint16)
    m = np.empty_like(sc)
    sc[..., 0:4] = s[..., 0:4] & 63
    m[..., 0:4] = s[..., 4:8] & 63
    sc[..., 4:8] = (s[..., 8:12] & 0x0F) | ((s[..., 0:4] >> 6) << 4)
    m[..., 4:8] = (s[..., 8:12] >> 4) | ((s[..., 4:8] >> 6) << 4)
    return sc, m


def dequant_q4_k(raw):
    b = _blocks(raw, Q4_K)
    nb = b.shape[0]
    d = _f16(b[:, 0:2])
    dmin = _f16(b[:, 2:4])
    sc, m = q4k_scales_mins(b[:, 4:16])
    qs = b[:, 16:144].reshape(nb, 4, 32)  # four 64-element chunks, 32 bytes each
    lo = (qs & 0x0F).astype(np.float64)  # sub-block 2c
    hi = (qs >> 4).astype(np.float64)  # sub-block 2c+1
    q = np.stack([lo, hi], axis=2).reshape(nb, 8, 32)  # sub-block major, 32 elems each
    y = (d[:, None, None] * sc[:, :, None].astype(np.float64)) * q - (dmin[:, None, None] * m[:, :, None].astype(np.float64))
    return y.astype(np.float32).reshape(-1)


def dequant_q6_k(raw):
    b = _blocks(raw, Q6_K)
    nb = b.shape[0]
    ql = b[:, 0:128].reshape(nb, 2, 2, 32)  # [half n][first/second 32 bytes][l]
    qh = b[:, 128:192].reshape(nb, 2, 32)  # [half n][l]
    sc = b[:, 192:208].view(np.int8).astype(np.float64).reshape(nb, 2, 8)  # [half n][8]
    d = _f16(b[:, 208:210])
    # quarter index r = 0..3 -> elements 128n + 32r + l
    lo4 = np.stack(
        [ql[:, :, 0, :] & 0x0F, ql[:, :, 1, :] & 0x0F, ql[:, :, 0, :] >> 4, ql[:, :, 1, :] >> 4], axis=2
    )  # [nb,2,4,32]
    hi2 = np.stack([(qh >> (2 * r)) & 3 for r in range(4)], axis=2)  # [nb,2,4,32]
    q = (lo4 | (hi2 << 4)).astype(np.int16) - 32
    # scale index = 2r + l // 16 within the half
    l_half = (np.arange(32) // 16)[None, None, None, :]
    r_idx = (2 * np.arange(4))[None, None, :, None]
    sidx = np.broadcast_to(r_idx + l_half, (nb, 2, 4, 32))
    s = np.take_along_axis(sc[:, :, None, :].repeat(4, axis=2), sidx, axis=3)
    y = d[:, None, None, None] * s * q.astype(np.float64)
    return y.astype(np.float32).reshape(-1)


# ---- the further formats (whole-array forms; unpinned by the reference like the three above) ------------

def _nibbles32(qs16):
    """[nb,16] bytes -> [nb,32] values: low nibbles are elements 0..15, high nibbles 16..31."""
    return np.concatenate([qs16 & 0x0F, qs16 >> 4], axis=1).astype(np.int32)


def _fifth_bits(qh4):
    """[nb,4] bytes of a little-endian u32 -> [nb,32] bits, bit j for element j."""
    qh = qh4.astype(np.uint32)
    word = qh[:, 0] | (qh[:, 1] << 8) | (qh[:, 2] << 16) | (qh[:, 3] << 24)
    return ((word[:, None] >> np.arange(32, dtype=np.uint32)[None, :]) & 1).astype(np.int32)


def dequant_q4_0(raw):
    b = _blocks(raw, Q4_0)
    return (_f16(b[:, 0:2])[:, None] * (_nibbles32(b[:, 2:18]) - 8)).astype(np.float32).reshape(-1)


def dequant_q4_1(raw):
    b = _blocks(raw, Q4_1)
    y = _f16(b[:, 0:2])[:, None] * _nibbles32(b[:, 4:20]) + _f16(b[:, 2:4])[:, None]
    return y.astype(np.float32).reshape(-1)


def dequant_q5_0(raw):
    b = _blocks(raw, Q5_0)
    q = (_nibbles32(b[:, 6:22]) | (_fifth_bits(b[:, 2:6]) << 4)) - 16
    return (_f16(b[:, 0:2])[:, None] * q).astype(np.float32).reshape(-1)


def dequant_q5_1(raw):
    b = _blocks(raw, Q5_1)
    q = _nibbles32(b[:, 8:24]) | (_fifth_bits(b[:, 4:8]) << 4)
    y = _f16(b[:, 0:2])[:, None] * q + _f16(b[:, 2:4])[:, None]
    return y.astype(np.float32).reshape(-1)


def dequant_q2_k(raw):
    b = _blocks(raw, Q2_K)
    nb = b.shape[0]
    s = b[:, 0:16].reshape(nb, 2, 4, 2)              # [half n][bit pair j][first / second 16 of the 32]
    qs = b[:, 16:80].reshape(nb, 2, 1, 32)           # [half n][.][l]
    shifts = (2 * np.arange(4, dtype=np.uint8)).reshape(1, 1, 4, 1)
    q = ((qs >> shifts) & 3).astype(np.float64)      # [nb,2,4,32]
    sc = np.repeat(s & 0x0F, 16, axis=3).astype(np.float64)   # [nb,2,4,32]
    mn = np.repeat(s >> 4, 16, axis=3).astype(np.float64)
    d = _f16(b[:, 80:82])[:, None, None, None]
    dmin = _f16(b[:, 82:84])[:, None, None, None]
    return ((d * sc) * q - dmin * mn).astype(np.float32).reshape(-1)


def dequant_q5_k(raw):
    b = _blocks(raw, Q5_K)
    nb = b.shape[0]
    d = _f16(b[:, 0:2])
    dmin = _f16(b[:, 2:4])
    sc, m = q4k_scales_mins(b[:, 4:16])
    qh = b[:, 16:48]                                  # [nb,32]
    qs = b[:, 48:176].reshape(nb, 4, 32)
    lo = (qs & 0x0F).astype(np.int32)
    hi = (qs >> 4).astype(np.int32)
    q = np.stack([lo, hi], axis=2).reshape(nb, 8, 32)  # sub-block j = 2c + upper
    bit = ((qh[:, None, :] >> np.arange(8, dtype=np.uint8)[None, :, None]) & 1).astype(np.int32)  # [nb,8,32]
    q = (q | (bit << 4)).astype(np.float64)
    y = (d[:, None, None] * sc[:, :, None].astype(np.float64)) * q - (dmin[:, None, None] * m[:, :, None].astype(np.float64))
    return y.astype(np.float32).reshape(-1)


def dequant_q3_k(raw):
    b = _blocks(raw, Q3_K)
    nb = b.shape[0]
    hm = b[:, 0:32]
    qs = b[:, 32:96].reshape(nb, 2, 1, 32)
    s = b[:, 96:108].astype(np.int32)
    low = np.concatenate([s[:, 0:8] & 0x0F, s[:, 0:8] >> 4], axis=1)                       # [nb,16]
    idx = np.arange(16)
    high = (s[:, 8 + idx % 4] >> (2 * (idx // 4))[None, :]) & 3                            # [nb,16]
    sc = ((low | (high << 4)) - 32).reshape(nb, 2, 4, 2)                                   # [half][pair][first / second 16]
    shifts = (2 * np.arange(4, dtype=np.uint8)).reshape(1, 1, 4, 1)
    q2 = ((qs >> shifts) & 3).astype(np.int32)                                             # [nb,2,4,32]
    bitpos = (4 * np.arange(2)[:, None] + np.arange(4)[None, :]).astype(np.uint8)          # [2,4]
    hbit = (hm[:, None, None, :] >> bitpos[None, :, :, None]) & 1                          # [nb,2,4,32]
    q = q2 - 4 * (1 - hbit.astype(np.int32))
    scale = np.repeat(sc, 16, axis=3).astype(np.float64)                                   # [nb,2,4,32]
    d = _f16(b[:, 108:110])[:, None, None, None]
    return (d * scale * q).astype(np.float32).reshape(-1)


def dequant_q8_k(raw):
    b = _blocks(raw, Q8_K)
    d = np.ascontiguousarray(b[:, 0:4]).view("<f4").astype(np.float64)                     # [nb,1]
    q = b[:, 4:260].view(np.int8).astype(np.float64)
    return (d * q).astype(np.float32).reshape(-1)


IQ4_VALUES = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], dtype=np.float64)


def dequant_iq4_nl(raw):
    b = _blocks(raw, IQ4_NL)
    return (_f16(b[:, 0:2])[:, None] * IQ4_VALUES[_nibbles32(b[:, 2:18])]).astype(np.float32).reshape(-1)


def dequant_iq4_xs(raw):
    b = _blocks(raw, IQ4_XS)
    nb = b.shape[0]
    sh = b[:, 2].astype(np.int32) | (b[:, 3].astype(np.int32) << 8)
    ib = np.arange(8)
    low = (b[:, 4 + ib // 2].astype(np.int32) >> (4 * (ib % 2))[None, :]) & 0x0F
    high = (sh[:, None] >> (2 * ib)[None, :]) & 3
    ls = ((low | (high << 4)) - 32).astype(np.float64)                                      # [nb,8]
    qs = b[:, 8:136].reshape(nb, 8, 16)
    vals = IQ4_VALUES[np.concatenate([qs & 0x0F, qs >> 4], axis=2).astype(np.int64)]       # [nb,8,32]
    return ((_f16(b[:, 0:2])[:, None] * ls)[:, :, None] * vals).astype(np.float32).reshape(-1)


def dequant_tq1_0(raw):
    """Five trits per byte (four in qh) as a base-3 fraction: trit n = ((byte * 3^n mod 256) * 3) >> 8."""
    b = _blocks(raw, TQ1_0)
    nb = b.shape[0]
    d = _f16(b[:, 52:54])

    def trits(bytes_, count):  # [nb, m] -> [nb, count, m]
        p3 = np.array([1, 3, 9, 27, 81], dtype=np.int64)[:count]
        q = (bytes_.astype(np.int64)[:, None, :] * p3[None, :, None]) & 0xFF
        return (q * 3) >> 8

    t = np.concatenate([trits(b[:, 0:32], 5).reshape(nb, 160), trits(b[:, 32:48], 5).reshape(nb, 80),
                        trits(b[:, 48:52], 4).reshape(nb, 16)], axis=1)
    return (d[:, None] * (t - 1).astype(np.float64)).astype(np.float32).reshape(-1)


def dequant_tq2_0(raw):
    b = _blocks(raw, TQ2_0)
    nb = b.shape[0]
    qs = b[:, 0:64].reshape(nb, 2, 1, 32).astype(np.int64)
    q = (qs >> (2 * np.arange(4))[None, None, :, None]) & 3                                  # [nb,2,4,32]
    return (_f16(b[:, 64:66])[:, None] * (q.reshape(nb, 256) - 1).astype(np.float64)).astype(np.float32).reshape(-1)


def dequant_f16(raw):
    return np.frombuffer(np.ascontiguousarray(raw), dtype="<f2").astype(np.float32)


def dequant_bf16(raw):
    return bf16_to_f32(np.frombuffer(np.ascontiguousarray(raw), dtype="<u2"))


def dequant_f32(raw):
    return np.frombuffer(np.ascontiguousarray(raw), dtype="<f4").copy()


_DEQ = {Q8_0: dequant_q8_0, Q4_K: dequant_q4_k, Q6_K: dequant_q6_k, Q4_0: dequant_q4_0, Q4_1: dequant_q4_1,
        Q5_0: dequant_q5_0, Q5_1: dequant_q5_1, Q2_K: dequant_q2_k, Q5_K: dequant_q5_k, F16: dequant_f16,
        Q3_K: dequant_q3_k, Q8_K: dequant_q8_k, IQ4_NL: dequant_iq4_nl, IQ4_XS: dequant_iq4_xs,
        TQ1_0: dequant_tq1_0, TQ2_0: dequant_tq2_0,
        BF16: dequant_bf16, F32: dequant_f32}


def dequant(qtype, raw):
    if qtype not in _DEQ:
        raise ValueError(f"unsupported ggml type {qtype}")
    return _DEQ[qtype](raw)


def matvec_q(qtype, raw, n_rows, k, x):
    """y = deq(W) . x with fp64 accumulation; the dense reduction of DoublesTensor.kt:255-264 on W^T."""
    quant_shape_to_byte_shape((n_rows, k), qtype)
    w = dequant(qtype, raw).reshape(n_rows, k).astype(np.float64)
    return (w @ np.asarray(x, dtype=np.float64)).astype(np.float32)


def bf16_to_f32(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(x):
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    return ((u + 0x7FFF + lsb) >> 16).astype(np.uint16)


def gemm_q(qtype, raw, n_rows, k, a_bf16, m):
    """C[m,n] = sum_k A[m,k] deq(W)[n,k], fp64 accumulation (DoublesTensor.kt:267-279 on W^T)."""
    w = dequant(qtype, raw).reshape(n_rows, k).astype(np.float64)
    a = bf16_to_f32(a_bf16).reshape(m, k).astype(np.float64)
    return (a @ w.T).astype(np.float32)


def dense_vecmat(x, b):
    """DoublesTensor.kt:255-264 including its shape error."""
    x = np.asarray(x, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    if x.shape[0] != b.shape[0]:
        raise ValueError("Shapes do not align.")
    y = np.zeros(b.shape[1])
    for i in range(x.shape[0]):
        y += x[i] * b[i]
    return y


def dense_matmul(a, b):
    """DoublesTensor.kt:267-279 including its shape error."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    if a.shape[1] != b.shape[0]:
        raise ValueError("Shapes do not align.")
    return a @ b


def linear(x, weight, bias):
    """Linear.kt:43-49: input.matmul(weight.t()) + bias with weight [out, in]."""
    w = np.asarray(weight, dtype=np.float64)
    x = np.asarray(x, dtype=np.float64)
    y = dense_vecmat(x, w.T) if x.ndim == 1 else dense_matmul(x, w.T)
    return y + np.asarray(bias, dtype=np.float64)


class FlatKV:
    """Shadow of the paged cache: plain [n_seq][max_tokens][n_head][dim] uint16 (fp16 bits) arrays."""

    def __init__(self, n_seq, n_head, dim, max_tokens):
        self.k = np.zeros((n_seq, max_tokens, n_head, dim), dtype=np.uint16)
        self.v = np.zeros_like(self.k)
        self.len = np.zeros(n_seq, dtype=np.int64)
        self.max_tokens = max_tokens

    def append(self, k_rows, v_rows, seq_ids):
        """k_rows, v_rows: [n][n_head][dim] fp16 bits; one token for each listed sequence, in order."""
        for i, s in enumerate(seq_ids):
            t = int(self.len[s])
            if t >= self.max_tokens:
                raise IndexError("sequence is full")
            self.k[s, t] = k_rows[i]
            self.v[s, t] = v_rows[i]
            self.len[s] = t + 1

    def gather(self, seq, t0, t1):
        return self.k[seq, t0:t1].copy(), self.v[seq, t0:t1].copy()


def attn_decode(q, k_bits, v_bits, n_ctx, scale):
    """q [S,H,D] fp32; k_bits/v_bits [S,T,H,D] fp16 bits; per-sequence context lengths -> out [S,H,D] fp32.

    Textbook max-subtracted softmax in fp64 (the reference's softmax, DoublesTensor.kt:392-395,491-519,
    is neither max-subtracted nor a softmax over the right axis and is untested there; it is not followed).
    """
    q = np.asarray(q, dtype=np.float64)
    out = np.zeros(q.shape, dtype=np.float32)
    for s in range(q.shape[0]):
        n = int(n_ctx[s])
        k = k_bits[s, :n].view(np.float16).astype(np.float64)  # [n,H,D]
        v = v_bits[s, :n].view(np.float16).astype(np.float64)
        sc = np.einsum("hd,thd->ht", q[s], k) * scale
        sc -= sc.max(axis=1, keepdims=True)
        p = np.exp(sc)
        p /= p.sum(axis=1, keepdims=True)
        out[s] = np.einsum("ht,thd->hd", p, v).astype(np.float32)
    return out


def rmsnorm(x, w, eps=1e-5):
    x = np.asarray(x, dtype=np.float64)
    r = 1.0 / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
    return (x * r * np.asarray(w, dtype=np.float64)).astype(np.float32)


def rope(x, pos, base=10000.0):
    """x [..., n_head, dim]; interleaved pairs (2i, 2i+1); angle = pos * base**(-2i/dim)."""
    x = np.asarray(x, dtype=np.float64).copy()
    dim = x.shape[-1]
    i = np.arange(dim // 2)
    theta = pos * base ** (-2.0 * i / dim)
    c, s = np.cos(theta), np.sin(theta)
    a, b = x[..., 0::2].copy(), x[..., 1::2].copy()
    x[..., 0::2] = a * c - b * s
    x[..., 1::2] = a * s + b * c
    return x.astype(np.float32)


def swiglu(gate, up):
    g = np.asarray(gate, dtype=np.float64)
    return (g / (1.0 + np.exp(-g)) * np.asarray(up, dtype=np.float64)).astype(np.float32)


def rel_err(actual, ref):
    """max_i |a_i - r_i| / max(|r_i|, 1e-3 * max|r|): the error metric every tolerance in the tests uses."""
    a = np.asarray(actual, dtype=np.float64).reshape(-1)
    r = np.asarray(ref, dtype=np.float64).reshape(-1)
    floor = 1e-3 * np.max(np.abs(r)) if r.size else 0.0
    den = np.maximum(np.abs(r), max(floor, 1e-300))
    return float(np.max(np.abs(a - r) / den)) if r.size else 0.0
