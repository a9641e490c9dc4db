#!/usr/bin/env python3
"""Writes the golden fixtures under tests/golden/.  Run from the repository root in the build container:

    python tests/golden/make_golden.py [--reference /root/reference]

Two kinds of fixture come out of it:

1. DATA the reference's own tests hold for this path (read as text / bytes, nothing is executed):
     tensor_test_vectors.json   the operands and expected results of the matmul known-answer tests in
                                core/src/commonTest/kotlin/sk/ai/net/TensorTest.kt (numbers only)
     test_experiment.gguf       gguf/src/jvmTest/resources/test_experiment.gguf (512-byte GGUF v3 container)
     sinus-approximator.json    io/src/jvmTest/resources/sinus-approximator.json (sine-MLP weights whose
                                end-to-end answer CsvParametersLoaderTest.kt:70 asserts)
   These need the reference checkout and are skipped (left as committed) when it is absent.

2. Seeded block vectors for the quantized formats (quant_blocks.npz): raw Q8_0 / Q4_K / Q6_K bytes from
   skainet_amd.synth plus adversarial hand-built blocks (fp16-subnormal and maximal scales, all-ones
   scale bytes, extreme int8), together with their dequantized values as computed by a slow, explicit,
   per-element Python evaluation in exact rational arithmetic (fractions.Fraction) rounded once to fp32.
   That evaluator is a third formulation beside oracle.c and oracle_np.py; the fixtures let both oracles
   and the GPU library be checked on boxes that have neither the reference nor this script's runtime.
"""
from __future__ import annotations

import argparse
import json
import os
import re
import shutil
import sys
from fractions import Fraction

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from skainet_amd import synth  # noqa: E402

NUM = r"-?\d+(?:\.\d+)?(?:[eE][-+]?\d+)?"


def _strip_comments(src):
    return re.sub(r"//[^\n]*", "", src)


def _tensors_in(body):
    """All createTensor(Shape(...), doubleArrayOf(...)) literals of a Kotlin test body, in order."""
    out = []
    for m in re.finditer(r"createTensor\(\s*(?:Shape\(([^)]*)\)\s*,\s*)?doubleArrayOf\(([^)]*)\)", body, re.S):
        shape = [int(s) for s in re.findall(r"\d+", m.group(1) or "")]
        vals = [float(v) for v in re.findall(NUM, m.group(2))]
        out.append({"shape": shape, "values": vals})
    return out


def _double_arrays_in(body):
    return [[float(v) for v in re.findall(NUM, m.group(1))] for m in re.finditer(r"(?<!createTensor\()doubleArrayOf\(([^)]*)\)", body, re.S)]


def extract_tensor_test(ref):
    path = os.path.join(ref, "core/src/commonTest/kotlin/sk/ai/net/TensorTest.kt")
    src = _strip_comments(open(path, encoding="utf-8").read())
    # split into test functions
    parts = re.split(r"@Test", src)
    cases = {}
    for p in parts:
        m = re.search(r"fun\s+(`[^`]+`|\w+)\s*\(", p)
        if not m:
            continue
        name = m.group(1).strip("`")
        if "matmul" not in name.lower():
            continue
        tensors = _tensors_in(p)
        expected = None
        em = re.search(r"assertContentEquals\(\s*doubleArrayOf\(([^)]*)\)", p, re.S)
        if em:
            expected = [float(v) for v in re.findall(NUM, em.group(1))]
        fm = re.search(r"val expected\w*\s*=\s*doubleArrayOf\(([^)]*)\)", p, re.S)
        if fm:
            expected = [float(v) for v in re.findall(NUM, fm.group(1))]
        msg = re.search(r'assertEquals\("([^"]+)",\s*exception\.message\)', p)
        cases[name] = {"tensors": tensors, "expected": expected, "error": msg.group(1) if msg else None}
    return {"source": "core/src/commonTest/kotlin/sk/ai/net/TensorTest.kt", "cases": cases}


# ---- exact per-element evaluator (third formulation) -------------------------------------------


def _f16_exact(lo, hi):
    bits = int(lo) | (int(hi) << 8)
    sign = -1 if bits & 0x8000 else 1
    e = (bits >> 10) & 0x1F
    m = bits & 0x3FF
    assert e != 31, "fixtures hold finite scales only"
    if e == 0:
        return sign * Fraction(m, 1 << 24)
    return sign * Fraction(1024 + m, 1024) * (Fraction(2) ** (e - 15))


def _round_f32(fr):
    """Fraction -> nearest binary32 (ties to even), in integer arithmetic; no intermediate binary64."""
    if fr == 0:
        return np.float32(0.0)
    sign = -1 if fr < 0 else 1
    a = abs(fr)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1  # now 2^e <= a < 2^(e+1)
    e = max(e, -126)  # subnormal range shares the exponent of the smallest normal
    scaled = a / (Fraction(2) ** (e - 23))  # the 24-bit significand as a rational
    n, rem = divmod(scaled.numerator, scaled.denominator)
    twice = 2 * rem
    if twice > scaled.denominator or (twice == scaled.denominator and (n & 1)):
        n += 1
    return np.float32(sign * float(n) * 2.0 ** (e - 23))


def _neg(lo, hi):
    return bool(int(hi) & 0x80)


def _zero(negative):
    return np.float32(-0.0) if negative else np.float32(0.0)


def exact_q8_0(b):
    d = _f16_exact(b[0], b[1])
    out = []
    for i in range(32):
        q = int(b[2 + i]) - 256 if b[2 + i] > 127 else int(b[2 + i])
        v = d * q
        # IEEE sign of an exact zero product: xor of the operand signs (the integer 0 converts to +0)
        out.append(_round_f32(v) if v != 0 else _zero(_neg(b[0], b[1]) ^ (q < 0)))
    return out


def exact_q4_k(b):
    d = _f16_exact(b[0], b[1])
    dmin = _f16_exact(b[2], b[3])
    s = [int(v) for v in b[4:16]]
    qs = [int(v) for v in b[16:144]]
    out = []
    for e in range(256):
        j = e // 32
        if j < 4:
            sc, m = s[j] & 63, s[j + 4] & 63
        else:
            sc = (s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4)
            m = (s[j + 4] >> 4) | ((s[j] >> 6) << 4)
        byte = qs[32 * (e // 64) + e % 32]
        q = (byte >> 4) if (e % 64) >= 32 else (byte & 15)
        v = d * sc * q - dmin * m
        if v != 0:
            out.append(_round_f32(v))
        else:
            # x - y with an exact zero result is +0 under round-to-nearest unless x is -0 and y is +0
            t1_negzero = (d * sc * q == 0) and _neg(b[0], b[1])
            t2_poszero = (dmin * m == 0) and not _neg(b[2], b[3])
            out.append(_zero(t1_negzero and t2_poszero))
    return out


def exact_q6_k(b):
    ql = [int(v) for v in b[0:128]]
    qh = [int(v) for v in b[128:192]]
    sc = [int(v) - 256 if v > 127 else int(v) for v in b[192:208]]
    d = _f16_exact(b[208], b[209])
    out = []
    for e in range(256):
        n, r = divmod(e, 128)
        quarter, l = divmod(r, 32)
        lo_byte = ql[64 * n + l + (32 if quarter in (1, 3) else 0)]
        lo = (lo_byte >> 4) if quarter >= 2 else (lo_byte & 15)
        hi = (qh[32 * n + l] >> (2 * quarter)) & 3
        q = (lo | (hi << 4)) - 32
        s = sc[8 * n + 2 * quarter + l // 16]
        v = d * s * q
        out.append(_round_f32(v) if v != 0 else _zero(_neg(b[208], b[209]) ^ (s < 0) ^ (q < 0)))
    return out


def _exact_affine(d, q, m, d_neg, m_bits=None):
    """d * q + m (m = None: no offset) as an exactly rounded float32 with IEEE zero signs."""
    v = d * q + (m if m is not None else 0)
    if v != 0:
        return _round_f32(v)
    prod_negzero = (d * q == 0) and (d_neg ^ (q < 0))
    if m is None:
        return _zero(prod_negzero)
    # x + y with an exact zero sum is +0 unless both are -0 (or x = -y != 0: +0)
    m_negzero = (m == 0) and _neg(*m_bits)
    return _zero(prod_negzero and m_negzero) if (d * q == 0 and m == 0) else _zero(False)


def _nibbles32(qs16):
    return [int(v) & 15 for v in qs16] + [int(v) >> 4 for v in qs16]


def exact_q4_0(b):
    d = _f16_exact(b[0], b[1])
    return [_exact_affine(d, q - 8, None, _neg(b[0], b[1])) for q in _nibbles32(b[2:18])]


def exact_q4_1(b):
    d, m = _f16_exact(b[0], b[1]), _f16_exact(b[2], b[3])
    return [_exact_affine(d, q, m, _neg(b[0], b[1]), (b[2], b[3])) for q in _nibbles32(b[4:20])]


def _qh_bits(b4):
    word = int(b4[0]) | (int(b4[1]) << 8) | (int(b4[2]) << 16) | (int(b4[3]) << 24)
    return [(word >> j) & 1 for j in range(32)]


def exact_q5_0(b):
    d = _f16_exact(b[0], b[1])
    q5 = [n | (h << 4) for n, h in zip(_nibbles32(b[6:22]), _qh_bits(b[2:6]))]
    return [_exact_affine(d, q - 16, None, _neg(b[0], b[1])) for q in q5]


def exact_q5_1(b):
    d, m = _f16_exact(b[0], b[1]), _f16_exact(b[2], b[3])
    q5 = [n | (h << 4) for n, h in zip(_nibbles32(b[8:24]), _qh_bits(b[4:8]))]
    return [_exact_affine(d, q, m, _neg(b[0], b[1]), (b[2], b[3])) for q in q5]


def _exact_scaled_minus(d, sc, q, dmin, m, d_bits, dmin_bits):
    v = d * sc * q - dmin * m
    if v != 0:
        return _round_f32(v)
    t1_negzero = (d * sc * q == 0) and _neg(*d_bits)
    t2_poszero = (dmin * m == 0) and not _neg(*dmin_bits)
    return _zero(t1_negzero and t2_poszero)


def exact_q2_k(b):
    d, dmin = _f16_exact(b[80], b[81]), _f16_exact(b[82], b[83])
    out = []
    for e in range(256):
        n, rem = divmod(e, 128)
        j, l = divmod(rem, 32)
        s = int(b[8 * n + 2 * j + (1 if l >= 16 else 0)])
        q = (int(b[16 + 32 * n + l]) >> (2 * j)) & 3
        out.append(_exact_scaled_minus(d, s & 15, q, dmin, s >> 4, (b[80], b[81]), (b[82], b[83])))
    return out


def exact_q5_k(b):
    d, dmin = _f16_exact(b[0], b[1]), _f16_exact(b[2], b[3])
    s = [int(v) for v in b[4:16]]
    out = []
    for e in range(256):
        j = e // 32
        if j < 4:
            sc, m = s[j] & 63, s[j + 4] & 63
        else:
            sc = (s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4)
            m = (s[j + 4] >> 4) | ((s[j] >> 6) << 4)
        byte = int(b[48 + 32 * (e // 64) + e % 32])
        q = ((byte >> 4) if (e % 64) >= 32 else (byte & 15)) | (((int(b[16 + e % 32]) >> j) & 1) << 4)
        out.append(_exact_scaled_minus(d, sc, q, dmin, m, (b[0], b[1]), (b[2], b[3])))
    return out


def _exact_product(d, factors, d_neg):
    """d times small integers as an exactly rounded float32; the zero keeps the xor of the operand signs."""
    v, neg = d, d_neg
    for f in factors:
        v *= f
        neg ^= f < 0
    return _round_f32(v) if v != 0 else _zero(neg)


def exact_q3_k(b):
    d = _f16_exact(b[108], b[109])
    s = [int(v) for v in b[96:108]]
    out = []
    for e in range(256):
        n, rem = divmod(e, 128)
        j, l = divmod(rem, 32)
        i = 8 * n + 2 * j + (1 if l >= 16 else 0)  # which of the sixteen scales
        lo4 = (s[i] & 15) if i < 8 else (s[i - 8] >> 4)
        hi2 = (s[8 + i % 4] >> (2 * (i // 4))) & 3
        q = (int(b[32 + 32 * n + l]) >> (2 * j)) & 3
        if not (int(b[l]) >> (4 * n + j)) & 1:
            q -= 4
        out.append(_exact_product(d, [(lo4 | (hi2 << 4)) - 32, q], _neg(b[108], b[109])))
    return out


def _f32_exact(b4):
    bits = int(b4[0]) | (int(b4[1]) << 8) | (int(b4[2]) << 16) | (int(b4[3]) << 24)
    sign = -1 if bits >> 31 else 1
    e, m = (bits >> 23) & 0xFF, bits & 0x7FFFFF
    assert e != 255, "fixtures hold finite scales only"
    if e == 0:
        return sign * Fraction(m, 1 << 149)
    return sign * Fraction((1 << 23) + m, 1 << 23) * (Fraction(2) ** (e - 127))


def exact_q8_k(b):
    d = _f32_exact(b[0:4])
    qs = [int(v) - 256 if v > 127 else int(v) for v in b[4:260]]
    return [_exact_product(d, [q], bool(int(b[3]) & 0x80)) for q in qs]


IQ4 = [-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113]


def exact_iq4_nl(b):
    d = _f16_exact(b[0], b[1])
    return [_exact_product(d, [IQ4[q]], _neg(b[0], b[1])) for q in _nibbles32(b[2:18])]


def exact_iq4_xs(b):
    d = _f16_exact(b[0], b[1])
    sh = int(b[2]) | (int(b[3]) << 8)
    out = []
    for ib in range(8):
        ls = ((int(b[4 + ib // 2]) >> (4 * (ib % 2))) & 15) | (((sh >> (2 * ib)) & 3) << 4)
        out += [_exact_product(d, [ls - 32, IQ4[q]], _neg(b[0], b[1])) for q in _nibbles32(b[8 + 16 * ib:24 + 16 * ib])]
    return out


def exact_tq1_0(b):
    """Independent of the multiply-and-shift decode: a byte is the base-3 fraction byte / 256, whose first five
    digits are the digits of floor(byte * 243 / 256)."""
    d = _f16_exact(b[52], b[53])
    neg = _neg(b[52], b[53])

    def trit(byte, n):
        return (int(byte) * 243 // 256) // 3 ** (4 - n) % 3

    out = [None] * 256
    for n in range(5):
        for m in range(32):
            out[32 * n + m] = _exact_product(d, [trit(b[m], n) - 1], neg)
        for m in range(16):
            out[160 + 16 * n + m] = _exact_product(d, [trit(b[32 + m], n) - 1], neg)
    for n in range(4):
        for j in range(4):
            out[240 + 4 * n + j] = _exact_product(d, [trit(b[48 + j], n) - 1], neg)
    return out


def exact_tq2_0(b):
    d = _f16_exact(b[64], b[65])
    neg = _neg(b[64], b[65])
    out = []
    for e in range(256):
        g, rem = divmod(e, 128)
        l, m = divmod(rem, 32)
        out.append(_exact_product(d, [((int(b[32 * g + m]) >> (2 * l)) & 3) - 1], neg))
    return out


EXACT = {synth.Q8_0: exact_q8_0, synth.Q4_K: exact_q4_k, synth.Q6_K: exact_q6_k}
EXACT_MORE = {synth.Q4_0: exact_q4_0, synth.Q4_1: exact_q4_1, synth.Q5_0: exact_q5_0, synth.Q5_1: exact_q5_1,
              synth.Q2_K: exact_q2_k, synth.Q5_K: exact_q5_k, synth.Q3_K: exact_q3_k, synth.Q8_K: exact_q8_k,
              synth.IQ4_NL: exact_iq4_nl, synth.IQ4_XS: exact_iq4_xs, synth.TQ1_0: exact_tq1_0,
              synth.TQ2_0: exact_tq2_0}
F16_FIELDS = {synth.Q4_0: (0,), synth.Q4_1: (0, 2), synth.Q5_0: (0,), synth.Q5_1: (0, 2), synth.Q2_K: (80, 82),
              synth.Q5_K: (0, 2), synth.Q3_K: (108,), synth.Q8_K: (), synth.IQ4_NL: (0,), synth.IQ4_XS: (0,),
              synth.TQ1_0: (52,), synth.TQ2_0: (64,)}
# Q8_K keeps its scale as a float32: subnormal, smallest normal, the largest whose products stay finite, odd significands, signed zeros
F32_EXTREMES = [0x00000001, 0x007FFFFF, 0x00800000, 0x7BFFFFFF, 0xBF800001, 0x3F800000, 0x00000000, 0x80000000,
                0x3DCCCCCD, 0xC2F6E979]


def adversarial_blocks(qtype, rng):
    """Blocks aimed at the places a restatement goes wrong: scale extremes, all-ones packing, sign bits."""
    _, bb = synth.BLOCK[qtype]
    blocks = []
    f16 = lambda v: list(np.array([v], dtype=np.float16).view(np.uint8))  # noqa: E731
    f16b = lambda bits: [bits & 0xFF, bits >> 8]  # noqa: E731
    scales16 = [f16b(0x0001), f16b(0x03FF), f16b(0x0400), f16b(0x7BFF), f16b(0x8001 | 0x3C00), f16(1.0), f16(0.0)]
    for sbytes in scales16:
        b = rng.integers(0, 256, size=bb, dtype=np.uint8)
        if qtype == synth.Q8_0:
            b[0:2] = sbytes
        elif qtype == synth.Q4_K:
            b[0:2] = sbytes
            b[2:4] = scales16[(scales16.index(sbytes) + 3) % len(scales16)]
        else:
            b[208:210] = sbytes
        blocks.append(b)
    # all-ones / all-zero packing bytes
    for fill in (0x00, 0xFF, 0x0F, 0xF0, 0x3F, 0xC0, 0x80, 0x7F):
        b = np.full(bb, fill, dtype=np.uint8)
        if qtype == synth.Q8_0:
            b[0:2] = f16(0.5)
        elif qtype == synth.Q4_K:
            b[0:2] = f16(0.25)
            b[2:4] = f16(0.125)
        else:
            b[208:210] = f16(-0.5)
        blocks.append(b)
    return np.stack(blocks).reshape(-1)


def make_quant_blocks():
    out = {}
    rng = np.random.default_rng(20240607)
    for qtype, name in ((synth.Q8_0, "q8_0"), (synth.Q4_K, "q4_k"), (synth.Q6_K, "q6_k")):
        be, bb = synth.BLOCK[qtype]
        n_rand = 24 if qtype == synth.Q8_0 else 6
        raw = np.concatenate([synth.weight(qtype, n_rand, be, seed=1000 + qtype), adversarial_blocks(qtype, rng)])
        blocks = raw.reshape(-1, bb)
        vals = np.array([EXACT[qtype](blk) for blk in blocks], dtype=np.float32).reshape(-1)
        out[f"{name}_raw"] = raw
        out[f"{name}_f32_bits"] = vals.view(np.uint32)
    np.savez_compressed(os.path.join(HERE, "quant_blocks.npz"), **out)
    return {k: v.shape for k, v in out.items()}


def make_more_quant_blocks():
    """The further formats: seeded blocks plus blocks with extreme fp16 fields and uniform fill bytes, evaluated
    exactly (rational arithmetic, rounded once); kept in their own fixture file."""
    out = {}
    rng = np.random.default_rng(20240611)
    names = {synth.Q4_0: "q4_0", synth.Q4_1: "q4_1", synth.Q5_0: "q5_0", synth.Q5_1: "q5_1", synth.Q2_K: "q2_k",
             synth.Q5_K: "q5_k", synth.Q3_K: "q3_k", synth.Q8_K: "q8_k", synth.IQ4_NL: "iq4_nl",
             synth.IQ4_XS: "iq4_xs", synth.TQ1_0: "tq1_0", synth.TQ2_0: "tq2_0"}
    f16b = lambda bits: [bits & 0xFF, bits >> 8]  # noqa: E731
    extremes = [f16b(0x0001), f16b(0x03FF), f16b(0x0400), f16b(0x7BFF), f16b(0xBC01), f16b(0x3C00), f16b(0x0000),
                f16b(0x8000)]
    for qtype, name in names.items():
        be, bb = synth.BLOCK[qtype]
        blocks = [synth.weight(qtype, 12 if be == 32 else 4, be, seed=2000 + qtype).reshape(-1, bb)]
        for i, ext in enumerate(extremes):
            b = rng.integers(0, 256, size=bb, dtype=np.uint8)
            for n, off in enumerate(F16_FIELDS[qtype]):
                b[off:off + 2] = extremes[(i + 3 * n) % len(extremes)]
            if qtype == synth.Q8_K:
                b[0:4] = np.array([F32_EXTREMES[i]], dtype="<u4").view(np.uint8)
            blocks.append(b[None, :])
        for fill in (0x00, 0xFF, 0x0F, 0xF0, 0x55, 0xAA):
            b = np.full(bb, fill, dtype=np.uint8)
            for n, off in enumerate(F16_FIELDS[qtype]):
                b[off:off + 2] = np.array([0.25 / (n + 1)], dtype=np.float16).view(np.uint8)
            if qtype == synth.Q8_K:
                b[0:4] = np.array([F32_EXTREMES[8 + (fill & 1)]], dtype="<u4").view(np.uint8)
            blocks.append(b[None, :])
        blocks = np.concatenate(blocks)
        vals = np.array([EXACT_MORE[qtype](blk) for blk in blocks], dtype=np.float32).reshape(-1)
        out[f"{name}_raw"] = blocks.reshape(-1)
        out[f"{name}_f32_bits"] = vals.view(np.uint32)
    np.savez_compressed(os.path.join(HERE, "quant_blocks_more.npz"), **out)
    return {k: v.shape for k, v in out.items()}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--reference", default="/root/reference")
    args = ap.parse_args()
    if os.path.isdir(args.reference):
        vec = extract_tensor_test(args.reference)
        with open(os.path.join(HERE, "tensor_test_vectors.json"), "w") as f:
            json.dump(vec, f, indent=1)
        print("tensor_test_vectors.json:", {k: (len(v["tensors"]), v["expected"] is not None) for k, v in vec["cases"].items()})
        for rel in ("gguf/src/jvmTest/resources/test_experiment.gguf", "io/src/jvmTest/resources/sinus-approximator.json"):
            shutil.copyfile(os.path.join(args.reference, rel), os.path.join(HERE, os.path.basename(rel)))
            os.chmod(os.path.join(HERE, os.path.basename(rel)), 0o644)
            print("copied", rel)
    else:
        print("reference checkout absent: keeping the committed reference-held fixtures")
    print("quant_blocks.npz:", make_quant_blocks())
    print("quant_blocks_more.npz:", make_more_quant_blocks())


if __name__ == "__main__":
    main()
