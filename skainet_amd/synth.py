"""Seeded synthetic GGUF block data of the benchmark shapes (NumPy, host side).

Every harness (tests, smoke, bench) draws its inputs from here so that the CPU oracle and the
GPU library always see identical bytes.  Layouts follow the ggml block definitions whose sizes
the reference tabulates in gguf/src/commonMain/kotlin/sk/ai/net/gguf/Constants.kt:58-90.

  Q8_0  34 B : f16 d = |N(0,1)|*0.02, 32 x int8 uniform in [-127, 127]
  Q4_K 144 B : f16 d = |N(0,1)|*0.01, f16 dmin = |N(0,1)|*0.005,
               12 bytes packing eight 6-bit scales and eight 6-bit mins (uniform 0..63),
               128 bytes of 4-bit quants (uniform 0..15)
  Q6_K 210 B : 128 B low nibbles + 64 B high 2-bit pairs (6-bit quants uniform 0..63),
               16 x int8 scales uniform in [-32, 31], f16 d = |N(0,1)|*0.01
"""
from __future__ import annotations

import numpy as np

Q8_0, Q4_K, Q6_K = 8, 12, 14
F32, F16, BF16 = 0, 1, 30
Q4_0, Q4_1, Q5_0, Q5_1, Q2_K, Q5_K = 2, 3, 6, 7, 10, 13
Q3_K, Q8_K, IQ4_NL, IQ4_XS = 11, 15, 20, 23
TQ1_0, TQ2_0 = 34, 35
BLOCK = {Q8_0: (32, 34), Q4_K: (256, 144), Q6_K: (256, 210), Q4_0: (32, 18), Q4_1: (32, 20), Q5_0: (32, 22),
         Q5_1: (32, 24), Q2_K: (256, 84), Q5_K: (256, 176), F32: (1, 4), F16: (1, 2), BF16: (1, 2),
         Q3_K: (256, 110), Q8_K: (256, 292), IQ4_NL: (32, 18), IQ4_XS: (256, 136), TQ1_0: (256, 54),
         TQ2_0: (256, 66)}


def _f16_bytes(values):
    return np.ascontiguousarray(values.astype(np.float16)).view(np.uint8).reshape(-1, 2)


def pack_q4k_scales(sc, m):
    """[nb,8] 6-bit scales and mins -> [nb,12] packed bytes (inverse of the ggml 6-bit unpack)."""
    sc = sc.astype(np.uint8)
    m = m.astype(np.uint8)
    out = np.empty(sc.shape[:-1] + (12,), dtype=np.uint8)
    out[..., 0:4] = (sc[..., 0:4] & 63) | ((sc[..., 4:8] >> 4) << 6)
    out[..., 4:8] = (m[..., 0:4] & 63) | ((m[..., 4:8] >> 4) << 6)
    out[..., 8:12] = (sc[..., 4:8] & 0x0F) | ((m[..., 4:8] & 0x0F) << 4)
    return out


def q8_0_blocks(n_blocks, rng):
    b = np.empty((n_blocks, 34), dtype=np.uint8)
    b[:, 0:2] = _f16_bytes(np.abs(rng.standard_normal(n_blocks)) * 0.02)
    b[:, 2:34] = rng.integers(-127, 128, size=(n_blocks, 32), dtype=np.int8).view(np.uint8)
    return b.reshape(-1)


def q4_k_blocks(n_blocks, rng):
    b = np.empty((n_blocks, 144), dtype=np.uint8)
    b[:, 0:2] = _f16_bytes(np.abs(rng.standard_normal(n_blocks)) * 0.01)
    b[:, 2:4] = _f16_bytes(np.abs(rng.standard_normal(n_blocks)) * 0.005)
    sc = rng.integers(0, 64, size=(n_blocks, 8), dtype=np.uint8)
    m = rng.integers(0, 64, size=(n_blocks, 8), dtype=np.uint8)
    b[:, 4:16] = pack_q4k_scales(sc, m)
    # two independent uniform nibbles per byte == one uniform byte
    b[:, 16:144] = rng.integers(0, 256, size=(n_blocks, 128), dtype=np.uint8)
    return b.reshape(-1)


def q6_k_blocks(n_blocks, rng):
    b = np.empty((n_blocks, 210), dtype=np.uint8)
    # 6-bit quants uniform 0..63 == uniform low nibble and uniform high 2 bits == uniform bytes
    b[:, 0:192] = rng.integers(0, 256, size=(n_blocks, 192), dtype=np.uint8)
    b[:, 192:208] = rng.integers(-32, 32, size=(n_blocks, 16), dtype=np.int8).view(np.uint8)
    b[:, 208:210] = _f16_bytes(np.abs(rng.standard_normal(n_blocks)) * 0.01)
    return b.reshape(-1)


def _scaled_blocks(n_blocks, rng, nbytes, f16_at, scale=0.01):
    """Uniform random payload bytes with |N(0,1)| * scale fp16 fields at the given byte offsets."""
    b = rng.integers(0, 256, size=(n_blocks, nbytes), dtype=np.uint8)
    for off in f16_at:
        b[:, off:off + 2] = _f16_bytes(np.abs(rng.standard_normal(n_blocks)) * scale)
    return b.reshape(-1)


def q5_k_blocks(n_blocks, rng):
    b = rng.integers(0, 256, size=(n_blocks, 176), dtype=np.uint8)
    b[:, 0:2] = _f16_bytes(np.abs(rng.standard_normal(n_blocks)) * 0.01)
    b[:, 2:4] = _f16_bytes(np.abs(rng.standard_normal(n_blocks)) * 0.005)
    b[:, 4:16] = pack_q4k_scales(rng.integers(0, 64, size=(n_blocks, 8), dtype=np.uint8),
                                 rng.integers(0, 64, size=(n_blocks, 8), dtype=np.uint8))
    return b.reshape(-1)


def q8_k_blocks(n_blocks, rng):
    b = rng.integers(0, 256, size=(n_blocks, 292), dtype=np.uint8)
    b[:, 0:4] = (np.abs(rng.standard_normal(n_blocks)) * 0.01).astype(np.float32).view(np.uint8).reshape(-1, 4)
    q = b[:, 4:260].view(np.int8).astype(np.int16).reshape(n_blocks, 16, 16)
    b[:, 260:292] = q.sum(axis=2).astype("<i2").view(np.uint8).reshape(n_blocks, 32)  # the block sums ggml keeps
    return b.reshape(-1)


def tq1_0_blocks(n_blocks, rng):
    """Valid encodings only: a byte is ceil(v * 256 / 243) for a five-trit value v (qh: four trits, then a zero)."""
    v = rng.integers(0, 243, size=(n_blocks, 52), dtype=np.int64)
    v[:, 48:52] = rng.integers(0, 81, size=(n_blocks, 4), dtype=np.int64) * 3
    b = np.empty((n_blocks, 54), dtype=np.uint8)
    b[:, 0:52] = ((v * 256 + 242) // 243).astype(np.uint8)
    b[:, 52:54] = _f16_bytes(np.abs(rng.standard_normal(n_blocks)) * 0.01)
    return b.reshape(-1)


def tq2_0_blocks(n_blocks, rng):
    q = rng.integers(0, 3, size=(n_blocks, 64, 4), dtype=np.uint8)  # two-bit fields hold 0..2
    b = np.empty((n_blocks, 66), dtype=np.uint8)
    b[:, 0:64] = q[:, :, 0] | (q[:, :, 1] << 2) | (q[:, :, 2] << 4) | (q[:, :, 3] << 6)
    b[:, 64:66] = _f16_bytes(np.abs(rng.standard_normal(n_blocks)) * 0.01)
    return b.reshape(-1)


_GEN = {
    TQ1_0: tq1_0_blocks,
    TQ2_0: tq2_0_blocks,
    Q3_K: lambda n, rng: _scaled_blocks(n, rng, 110, (108,)),
    Q8_K: q8_k_blocks,
    IQ4_NL: lambda n, rng: _scaled_blocks(n, rng, 18, (0,)),
    IQ4_XS: lambda n, rng: _scaled_blocks(n, rng, 136, (0,)),
    Q8_0: q8_0_blocks, Q4_K: q4_k_blocks, Q6_K: q6_k_blocks, Q5_K: q5_k_blocks,
    Q4_0: lambda n, rng: _scaled_blocks(n, rng, 18, (0,)),
    Q4_1: lambda n, rng: _scaled_blocks(n, rng, 20, (0, 2)),
    Q5_0: lambda n, rng: _scaled_blocks(n, rng, 22, (0,)),
    Q5_1: lambda n, rng: _scaled_blocks(n, rng, 24, (0, 2)),
    Q2_K: lambda n, rng: _scaled_blocks(n, rng, 84, (80, 82)),
    F32: lambda n, rng: rng.standard_normal(n, dtype=np.float32).view(np.uint8),
    F16: lambda n, rng: rng.standard_normal(n, dtype=np.float32).astype(np.float16).view(np.uint8),
    BF16: lambda n, rng: f32_to_bf16_bits(rng.standard_normal(n, dtype=np.float32)).view(np.uint8),
}


def weight(qtype, n_rows, k, seed):
    """Raw block bytes of an [n_rows, k] weight ([out, in], rows contiguous), as uint8."""
    elems, _ = BLOCK[qtype]
    if k % elems:
        raise ValueError(f"row size {k} is not a multiple of the block size {elems}")
    rng = np.random.default_rng(seed)
    return _GEN[qtype](n_rows * (k // elems), rng)


def activation_f32(n, seed):
    return np.random.default_rng(seed).standard_normal(n, dtype=np.float32)


def f32_to_bf16_bits(x):
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def activation_bf16(shape, seed):
    x = np.random.default_rng(seed).standard_normal(shape, dtype=np.float32)
    return f32_to_bf16_bits(x)


def kv_f16(shape, seed):
    """fp16 bit patterns of N(0,1) draws."""
    x = np.random.default_rng(seed).standard_normal(shape, dtype=np.float32)
    return x.astype(np.float16).view(np.uint16)


def checksum(arr):
    """FNV-1a 64 over a strided sample of the bytes plus the length: recorded beside bench results."""
    a = np.ascontiguousarray(arr).view(np.uint8).reshape(-1)
    step = max(1, a.size // 65536)
    h = 0xCBF29CE484222325
    for byte in a[::step].tolist():
        h = ((h ^ byte) * 0x100000001B3) & 0xFFFFFFFFFFFFFFFF
    return f"{h:016x}:{a.size}"


# ---- conditioned weights -------------------------------------------------------------------------------------
# The benchmark's Q4_K draws (d * sc * q - dmin * m with independent scales and minima) have a positive mean about
# two thirds of their spread: stacked into a decoder they drown the attention path in the feed-forward output.  The
# generator below keeps the block formats and their full field ranges but centres the values on zero and scales
# every d by a power of two, so that a matrix maps a unit-rms vector to a vector of a chosen rms ("gain").  It is
# what decoder tests use when the result must depend on positions, cache contents and attention.

# rms of a weight drawn by the base generators after centring, per format, at their stated d scales
# (Q8_0: d * q, q uniform in [-127, 127], d = |N| * 0.02; Q6_K: d * sc * (q - 32); the offset formats centred as below)
_CENTRED_RMS = {Q8_0: 1.4722, Q6_K: 3.4150, Q4_K: 1.6834, Q5_K: 3.3717, Q4_0: 0.046368, Q5_0: 0.092466}
_D_FIELDS = {Q8_0: (34, (0,)), Q6_K: (210, (208,)), Q4_K: (144, (0, 2)), Q5_K: (176, (0, 2)), Q4_0: (18, (0,)),
             Q5_0: (22, (0,))}


def conditioned_weight(qtype, n_rows, k, seed, gain=1.0):
    """Raw block bytes of an [n_rows, k] weight whose values are centred on zero and whose rows map a unit-rms
    vector to outputs of rms about `gain` (to the nearest power of two in d).  Q4_K / Q5_K: every sub-block gets
    m = sc and the superblock dmin = f16(7.5 d) / f16(15.5 d), i.e. values d * sc * (q - 7.5) / (q - 15.5)."""
    if qtype not in _CENTRED_RMS:
        raise ValueError(f"no conditioned generator for ggml type {qtype}")
    raw = weight(qtype, n_rows, k, seed)
    nbytes, d_at = _D_FIELDS[qtype]
    b = raw.reshape(-1, nbytes).copy()
    factor = 2.0 ** np.round(np.log2(gain / (_CENTRED_RMS[qtype] * np.sqrt(k))))
    d = b[:, d_at[0]:d_at[0] + 2].copy().view(np.float16).astype(np.float32).reshape(-1) * np.float32(factor)
    b[:, d_at[0]:d_at[0] + 2] = _f16_bytes(d)
    if qtype in (Q4_K, Q5_K):
        d = b[:, 0:2].copy().view(np.float16).astype(np.float32).reshape(-1)  # as stored
        b[:, 2:4] = _f16_bytes(d * np.float32(7.5 if qtype == Q4_K else 15.5))
        packed = b[:, 4:16]
        sc = np.empty((b.shape[0], 8), dtype=np.uint8)  # the scales as drawn; the minima become copies of them
        sc[:, 0:4] = packed[:, 0:4] & 63
        sc[:, 4:8] = (packed[:, 8:12] & 0x0F) | ((packed[:, 0:4] >> 6) << 4)
        b[:, 4:16] = pack_q4k_scales(sc, sc)
    return b.reshape(-1)


# ---- the library's generator, restated ------------------------------------------------------------------------
# skn_synth_* (csrc/synth.hip) produce the benchmark inputs inside the library so that C, ctypes and Kotlin harnesses
# draw identical bytes.  The functions below are the same algorithm in NumPy -- counter-based SplitMix64 words, integer
# arithmetic up to the final conversion -- and tests/test_synth_abi.py holds the two equal byte for byte.

_G = np.uint64(0x9E3779B97F4A7C15)


def _mix(z):
    z = np.asarray(z, dtype=np.uint64)
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def _words(seed, stream, first, count):
    """Words first .. first + count - 1 of a stream."""
    with np.errstate(over="ignore"):
        base = _mix(np.array([seed], dtype=np.uint64) + _G * np.uint64(stream + 1))[0]
        idx = np.arange(first + 1, first + count + 1, dtype=np.uint64)
        return _mix(base + _G * idx)


def _stream_bytes(seed, stream, n):
    return _words(seed, stream, 0, (n + 7) // 8).astype("<u8").view(np.uint8)[:n]


def _stream_normal(seed, stream, n):
    w = _words(seed, stream, 0, 6 * n).reshape(n, 6)
    total = ((w & np.uint64(0xFFFFFFFF)) + (w >> np.uint64(32))).sum(axis=1, dtype=np.uint64)
    return (total.astype(np.int64) - np.int64(6 << 32)).astype(np.float64) * (1.0 / 4294967296.0)


def _f16_via_f32(values):
    return np.ascontiguousarray(values.astype(np.float32).astype(np.float16)).view(np.uint8).reshape(-1, 2)


def lib_weight(qtype, n_rows, k, seed):
    """What skn_synth_weight writes: raw blocks of an [n_rows, k] Q8_0 / Q4_K / Q6_K weight."""
    if qtype not in (Q8_0, Q4_K, Q6_K):
        raise ValueError(f"ggml type {qtype} has no generator (Q8_0, Q4_K, Q6_K)")
    elems, nbytes = BLOCK[qtype]
    if k % elems:
        raise ValueError(f"row size {k} is not a multiple of the block size {elems}")
    nb = n_rows * (k // elems)
    b = np.empty((nb, nbytes), dtype=np.uint8)
    if nb == 0:
        return b.reshape(-1)
    if qtype == Q8_0:
        b[:, 0:2] = _f16_via_f32(np.abs(_stream_normal(seed, 1, nb)) * 0.02)
        u = _stream_bytes(seed, 0, 64 * nb).reshape(nb, 32, 2).astype(np.uint32)
        u16 = u[:, :, 0] | (u[:, :, 1] << 8)
        b[:, 2:34] = (((u16 * 255) >> 16).astype(np.int32) - 127).astype(np.int8).view(np.uint8)
    elif qtype == Q4_K:
        b[:, 0:2] = _f16_via_f32(np.abs(_stream_normal(seed, 1, nb)) * 0.01)
        b[:, 2:4] = _f16_via_f32(np.abs(_stream_normal(seed, 2, nb)) * 0.005)
        v = _stream_bytes(seed, 3, 16 * nb).reshape(nb, 16) & 63
        b[:, 4:16] = pack_q4k_scales(v[:, 0:8], v[:, 8:16])
        b[:, 16:144] = _stream_bytes(seed, 0, 128 * nb).reshape(nb, 128)
    else:
        b[:, 0:192] = _stream_bytes(seed, 0, 192 * nb).reshape(nb, 192)
        v = _stream_bytes(seed, 3, 16 * nb).reshape(nb, 16) & 63
        b[:, 192:208] = (v.astype(np.int16) - 32).astype(np.int8).view(np.uint8)
        b[:, 208:210] = _f16_via_f32(np.abs(_stream_normal(seed, 1, nb)) * 0.01)
    return b.reshape(-1)


def lib_activation_f32(n, seed):
    return _stream_normal(seed, 0, n).astype(np.float32)


def lib_activation_bf16(n, seed):
    return f32_to_bf16_bits(lib_activation_f32(n, seed))


def lib_kv_f16(n, seed):
    return lib_activation_f32(n, seed).astype(np.float16).view(np.uint16)


def lib_checksum(arr):
    """FNV-1a 64 over every byte (skn_synth_checksum); vectorised: h_n = (h_(n-1) ^ b_n) * P has no closed form, so
    this walks the bytes in Python and is meant for small buffers."""
    h = 0xCBF29CE484222325
    for byte in np.ascontiguousarray(arr).view(np.uint8).reshape(-1).tolist():
        h = ((h ^ byte) * 0x100000001B3) & 0xFFFFFFFFFFFFFFFF
    return h
