"""CPU: the two oracles against the golden block vectors, hand-built known answers and each other."""
import os

import numpy as np
import pytest

from oracle import oracle_c, oracle_np
from skainet_amd import synth

Q8_0, Q4_K, Q6_K = 8, 12, 14
TYPES = [(Q8_0, "q8_0"), (Q4_K, "q4_k"), (Q6_K, "q6_k")]


def f16_bytes(v):
    return np.array([v], dtype=np.float16).view(np.uint8)


@pytest.fixture(scope="module")
def blocks(golden_dir):
    return np.load(os.path.join(golden_dir, "quant_blocks.npz"))


def test_type_table_matches_reference_constants():
    # literal numbers of reference gguf/.../Constants.kt:65,69,71 and the enum ids :21,25,27
    assert oracle_c.type_sizes(8) == (32, 34)
    assert oracle_c.type_sizes(12) == (256, 144)
    assert oracle_c.type_sizes(14) == (256, 210)
    assert oracle_np.QUANT_SIZES[8] == (32, 34)
    assert oracle_np.QUANT_SIZES[12] == (256, 144)
    assert oracle_np.QUANT_SIZES[14] == (256, 210)
    with pytest.raises(ValueError):
        oracle_c.type_sizes(99)


def test_row_bytes_rule():
    # reference gguf/.../Quants.kt:10-20; the byte rows of the benchmark shapes
    assert oracle_c.row_bytes(Q4_K, 4096) == 2304
    assert oracle_c.row_bytes(Q4_K, 11008) == 6192
    assert oracle_c.row_bytes(Q8_0, 4096) == 4352
    assert oracle_c.row_bytes(Q6_K, 4096) == 3360
    assert oracle_c.row_bytes(Q4_K, 4100) == -3
    assert oracle_np.quant_shape_to_byte_shape((11008, 4096), Q4_K) == (11008, 2304)
    with pytest.raises(ValueError, match=r"Quantized tensor row size \(4100\) is not a multiple of Q4_K block size \(256\)"):
        oracle_np.quant_shape_to_byte_shape((2, 4100), Q4_K)


def test_h2f_all_65536_against_numpy():
    bits = np.arange(65536, dtype=np.uint16)
    mine = oracle_c.h2f(bits).view(np.uint32)
    ref = bits.view(np.float16).astype(np.float32).view(np.uint32)
    nan = np.isnan(bits.view(np.float16))
    assert np.array_equal(mine[~nan], ref[~nan])
    assert np.all(np.isnan(mine.view(np.float32)[nan]))


def test_f2h_round_to_nearest_even_against_numpy():
    rng = np.random.default_rng(1)
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 5, 200000).astype(np.float32),
        np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)[~np.isnan(np.arange(65536, dtype=np.uint16).view(np.float16))],
        np.array([65504.0, 65519.9, 65520.0, 1e9, 2.0 ** -25, 2.0 ** -25 * 1.0001, 2.0 ** -24 * 1.5, 2.0 ** -24 * 2.5, 0.0, -0.0], dtype=np.float32),
    ])
    with np.errstate(over="ignore"):
        ref = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle_c.f2h(x), ref)


@pytest.mark.parametrize("qtype,name", TYPES)
def test_oracles_match_golden_blocks(blocks, qtype, name):
    raw = blocks[f"{name}_raw"]
    want = blocks[f"{name}_f32_bits"]
    assert np.array_equal(oracle_c.dequant(qtype, raw).view(np.uint32), want)
    assert np.array_equal(oracle_np.dequant(qtype, raw).view(np.uint32), want)


@pytest.mark.parametrize("qtype,name", TYPES)
def test_oracles_agree_bitwise_on_random_blocks(qtype, name):
    be, bb = synth.BLOCK[qtype]
    raw = synth.weight(qtype, 64, 8 * be if be == 256 else 64 * be, seed=7 + qtype)
    a = oracle_c.dequant(qtype, raw)
    b = oracle_np.dequant(qtype, raw)
    assert a.size == raw.size // bb * be
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    # fully random bytes too (random f16 scales incl. subnormals; inf/nan scales excluded)
    rng = np.random.default_rng(99 + qtype)
    rnd = rng.integers(0, 256, size=(512, bb), dtype=np.uint8)
    pos = {Q8_0: [1], Q4_K: [1, 3], Q6_K: [209]}[qtype]
    for p in pos:
        rnd[:, p] &= 0x7B | 0x80  # clear one exponent bit: no inf / nan
    a = oracle_c.dequant(qtype, rnd.reshape(-1))
    b = oracle_np.dequant(qtype, rnd.reshape(-1))
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_q4k_known_answers():
    blk = np.zeros(144, dtype=np.uint8)
    blk[0:2] = f16_bytes(1.0)
    blk[2:4] = f16_bytes(0.5)
    # scales sc_j = j + 1, mins m_j = 2j + 3, through the published 6-bit packing written out by hand
    sc = [1, 2, 3, 4, 5, 6, 7, 8]
    m = [3, 5, 7, 9, 11, 13, 15, 17]
    s = blk[4:16]
    for j in range(4):
        s[j] = sc[j] | ((sc[j + 4] >> 4) << 6)
        s[j + 4] = m[j] | ((m[j + 4] >> 4) << 6)
        s[j + 8] = (sc[j + 4] & 15) | ((m[j + 4] & 15) << 4)
    # all quants zero -> y = -dmin * m_j on sub-block j
    y = oracle_c.dequant(Q4_K, blk)
    for j in range(8):
        assert np.all(y[32 * j:32 * j + 32] == -0.5 * m[j])
    # element order: byte i of chunk c carries element 64c+i (low nibble) and 64c+32+i (high nibble)
    blk[2:4] = f16_bytes(0.0)
    qs = blk[16:144].reshape(4, 32)
    for c in range(4):
        for i in range(32):
            lo, hi = (c + i) % 16, (3 * i + c + 5) % 16
            qs[c, i] = lo | (hi << 4)
    y = oracle_c.dequant(Q4_K, blk)
    for c in range(4):
        for i in range(32):
            assert y[64 * c + i] == sc[2 * c] * ((c + i) % 16)
            assert y[64 * c + 32 + i] == sc[2 * c + 1] * ((3 * i + c + 5) % 16)
    assert np.array_equal(oracle_np.dequant(Q4_K, blk), y)


def test_q4k_scale_unpack_with_high_bits():
    # sc/m >= 16 on sub-blocks 4..7 exercise the two bits parked in the top of bytes 0..7
    sc = np.array([[63, 0, 21, 42, 63, 16, 47, 32]], dtype=np.uint8)
    m = np.array([[0, 63, 42, 21, 48, 63, 15, 17]], dtype=np.uint8)
    packed = synth.pack_q4k_scales(sc, m)
    got_sc, got_m = oracle_np.q4k_scales_mins(packed)
    assert np.array_equal(got_sc, sc) and np.array_equal(got_m, m)
    blk = np.zeros(144, dtype=np.uint8)
    blk[0:2] = f16_bytes(1.0)
    blk[2:4] = f16_bytes(1.0)
    blk[4:16] = packed[0]
    blk[16:144] = 0x11  # every quant = 1 -> y = sc_j - m_j
    y = oracle_c.dequant(Q4_K, blk)
    for j in range(8):
        assert np.all(y[32 * j:32 * j + 32] == float(sc[0, j]) - float(m[0, j]))


def test_q6k_known_answers():
    blk = np.zeros(210, dtype=np.uint8)
    blk[208:210] = f16_bytes(1.0)
    blk[192:208] = np.arange(1, 17, dtype=np.int8).view(np.uint8)
    # quant code 32 (low nibble 0, high pair 2) is the zero point
    blk[0:128] = 0x00
    blk[128:192] = 0xAA
    assert np.all(oracle_c.dequant(Q6_K, blk) == 0.0)
    # code 33 everywhere -> y = scale of the 16-element group, groups in element order
    blk[0:128] = 0x11
    y = oracle_c.dequant(Q6_K, blk)
    for g in range(16):
        assert np.all(y[16 * g:16 * g + 16] == g + 1)
    # element order: tag each element with its own 6-bit code and unit scales
    blk[192:208] = 1
    codes = (np.arange(256) * 7 + 3) % 64
    ql = blk[0:128]
    qh = blk[128:192]
    ql[:] = 0
    qh[:] = 0
    for e in range(256):
        n, r = divmod(e, 128)
        quarter, l = divmod(r, 32)
        lo, hi = codes[e] & 15, codes[e] >> 4
        ql[64 * n + l + 32 * (quarter & 1)] |= lo << (4 * (quarter >> 1))
        qh[32 * n + l] |= hi << (2 * quarter)
    y = oracle_c.dequant(Q6_K, blk)
    assert np.array_equal(y, (codes - 32).astype(np.float32))
    assert np.array_equal(oracle_np.dequant(Q6_K, blk), y)


def test_q8_0_known_answers():
    blk = np.zeros(34, dtype=np.uint8)
    blk[0:2] = f16_bytes(0.25)
    blk[2:34] = np.arange(-16, 16, dtype=np.int8).view(np.uint8)
    y = oracle_c.dequant(Q8_0, blk)
    assert np.array_equal(y, np.arange(-16, 16, dtype=np.float32) * 0.25)
    blk[2:34] = np.int8(-128).view(np.uint8)
    assert np.all(oracle_np.dequant(Q8_0, blk) == -32.0)


def test_dequant_rejects_bad_arguments():
    with pytest.raises(ValueError):
        oracle_c.dequant(16, np.zeros(66, dtype=np.uint8), 256)  # IQ2_XXS: in the size table, not computed with
    with pytest.raises(ValueError):
        oracle_c.dequant(Q4_K, np.zeros(144, dtype=np.uint8), 100)
    with pytest.raises(ValueError):
        oracle_np.dequant(16, np.zeros(66, dtype=np.uint8))


def test_synthetic_generator_statistics():
    # the generator's own contract: scale magnitudes and value ranges of the benchmark configs
    raw = synth.weight(Q4_K, 64, 4096, seed=3).reshape(-1, 144)
    d = raw[:, 0:2].copy().view(np.float16).astype(np.float64)
    dmin = raw[:, 2:4].copy().view(np.float16).astype(np.float64)
    assert abs(d.mean() - 0.01 * np.sqrt(2 / np.pi)) < 5e-4
    assert abs(dmin.mean() - 0.005 * np.sqrt(2 / np.pi)) < 3e-4
    sc, m = oracle_np.q4k_scales_mins(raw[:, 4:16])
    assert sc.max() == 63 and sc.min() == 0 and m.max() == 63
    raw6 = synth.weight(Q6_K, 16, 4096, seed=4).reshape(-1, 210)
    s6 = raw6[:, 192:208].view(np.int8)
    assert s6.min() == -32 and s6.max() == 31
    raw8 = synth.weight(Q8_0, 16, 4096, seed=5).reshape(-1, 34)
    q8 = raw8[:, 2:].view(np.int8)
    assert q8.min() == -127 and q8.max() == 127
    assert np.array_equal(synth.weight(Q4_K, 4, 512, seed=11), synth.weight(Q4_K, 4, 512, seed=11))
