"""CPU: the further ggml block formats of the reference's size table (Constants.kt:58-90) -- Q4_0, Q4_1, Q5_0, Q5_1,
Q2_K, Q3_K, Q5_K, Q8_K, IQ4_NL, IQ4_XS, TQ1_0, TQ2_0, F16, BF16.  The reference holds only their sizes; the packing is the published ggml definition
(parity unpinned by the reference).  Pinned here by hand-built single blocks whose answers are known in closed
form (every field tagged so that a wrong element order, bit position or scale index shows), and by bit-for-bit
agreement of the two independently written oracles on random bytes."""
import numpy as np
import pytest

from oracle import oracle_c, oracle_np
from skainet_amd import synth

Q4_0, Q4_1, Q5_0, Q5_1, Q2_K, Q5_K = 2, 3, 6, 7, 10, 13
Q3_K, Q8_K, IQ4_NL, IQ4_XS = 11, 15, 20, 23
TQ1_0, TQ2_0 = 34, 35
F32, F16, BF16 = 0, 1, 30
MORE = [(Q4_0, "q4_0"), (Q4_1, "q4_1"), (Q5_0, "q5_0"), (Q5_1, "q5_1"), (Q2_K, "q2_k"), (Q5_K, "q5_k"),
        (Q3_K, "q3_k"), (Q8_K, "q8_k"), (IQ4_NL, "iq4_nl"), (IQ4_XS, "iq4_xs"), (TQ1_0, "tq1_0"), (TQ2_0, "tq2_0"),
        (F16, "f16"), (BF16, "bf16"), (F32, "f32")]
IQ4 = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], dtype=np.float64)


def f16b(v):
    return np.array([v], dtype=np.float16).view(np.uint8)


def both(qtype, raw):
    a = oracle_c.dequant(qtype, raw)
    b = oracle_np.dequant(qtype, raw)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    return a


@pytest.mark.parametrize("qtype,name", [t for t in MORE if t[0] not in (F16, BF16, F32)])
def test_oracles_match_golden_blocks(golden_dir, qtype, name):
    """tests/golden/quant_blocks_more.npz: a third formulation (exact rational arithmetic, rounded once) on seeded
    blocks, extreme fp16 fields (subnormal, largest, signed zero) and uniform fill bytes."""
    import os
    g = np.load(os.path.join(golden_dir, "quant_blocks_more.npz"))
    raw, want = g[f"{name}_raw"], g[f"{name}_f32_bits"]
    assert np.array_equal(oracle_c.dequant(qtype, raw).view(np.uint32), want)
    assert np.array_equal(oracle_np.dequant(qtype, raw).view(np.uint32), want)


def test_sizes_match_reference_table():
    # literal numbers of reference gguf/.../Constants.kt:60-90 and the enum ids :16-48
    want = {Q4_0: (32, 18), Q4_1: (32, 20), Q5_0: (32, 22), Q5_1: (32, 24), Q2_K: (256, 84), Q5_K: (256, 176),
            Q3_K: (256, 110), Q8_K: (256, 292), IQ4_NL: (32, 18), IQ4_XS: (256, 136), TQ1_0: (256, 54),
            TQ2_0: (256, 66), F16: (1, 2), BF16: (1, 2), F32: (1, 4)}
    for t, sz in want.items():
        assert oracle_c.type_sizes(t) == sz
        assert oracle_np.QUANT_SIZES[t] == sz
        assert synth.BLOCK[t] == sz


@pytest.mark.parametrize("qtype,name", MORE)
def test_oracles_agree_bitwise_on_random_blocks(qtype, name):
    be, bb = synth.BLOCK[qtype]
    rng = np.random.default_rng(qtype + 100)
    raw = rng.integers(0, 256, size=64 * bb, dtype=np.uint8)
    if qtype in (F16, BF16, F32):  # random bytes would hold NaNs: compare finite synthetic values instead
        raw = synth.weight(qtype, 4, 64, seed=3)
    else:
        # keep the fp16 fields finite (exponent field 31 is inf / nan)
        for off in {Q4_0: (0,), Q4_1: (0, 2), Q5_0: (0,), Q5_1: (0, 2), Q2_K: (80, 82), Q5_K: (0, 2), Q3_K: (108,),
                    Q8_K: (2,), IQ4_NL: (0,), IQ4_XS: (0,), TQ1_0: (52,), TQ2_0: (64,)}[qtype]:
            raw.reshape(-1, bb)[:, off + 1] &= 0x7B  # (Q8_K: the top byte of its float32 scale)
    both(qtype, raw)


def test_q4_0_and_q4_1_element_order():
    qs = np.array([j | ((15 - j) << 4) for j in range(16)], dtype=np.uint8)
    y = both(Q4_0, np.concatenate([f16b(2.0), qs]))
    assert np.array_equal(y[:16], 2.0 * (np.arange(16) - 8))        # low nibbles first
    assert np.array_equal(y[16:], 2.0 * ((15 - np.arange(16)) - 8))  # then high nibbles
    y = both(Q4_1, np.concatenate([f16b(0.5), f16b(-3.0), qs]))
    assert np.array_equal(y[:16], 0.5 * np.arange(16) - 3.0)
    assert np.array_equal(y[16:], 0.5 * (15 - np.arange(16)) - 3.0)


def test_q5_0_and_q5_1_fifth_bit_positions():
    qs = np.zeros(16, dtype=np.uint8)
    for bit in (0, 3, 15, 16, 20, 31):
        qh = np.array([(1 << bit) >> (8 * i) & 0xFF for i in range(4)], dtype=np.uint8)
        y = both(Q5_0, np.concatenate([f16b(1.0), qh, qs]))
        want = np.full(32, -16.0)
        want[bit] = 0.0  # bit j of qh is the fifth bit of element j
        assert np.array_equal(y, want), bit
        y = both(Q5_1, np.concatenate([f16b(1.0), f16b(0.25), qh, qs]))
        want = np.full(32, 0.25)
        want[bit] = 16.25
        assert np.array_equal(y, want), bit
    qs = np.arange(16, dtype=np.uint8) | ((15 - np.arange(16, dtype=np.uint8)) << 4)
    y = both(Q5_0, np.concatenate([f16b(1.0), np.array([0xFF, 0xFF, 0, 0], dtype=np.uint8), qs]))
    assert np.array_equal(y[:16], np.arange(16) + 16.0 - 16.0)
    assert np.array_equal(y[16:], (15 - np.arange(16)) - 16.0)


def test_q2_k_scale_index_and_bit_pairs():
    # scale nibble of group g is g % 16 with min 0: y = d * (g % 16) * q; every byte holds q = 1,2,3,0 in its
    # bit pairs 0..3, so element e reads q = [1,2,3,0][(e % 128) // 32]
    scales = np.arange(16, dtype=np.uint8)
    qs = np.full(64, 1 | (2 << 2) | (3 << 4) | (0 << 6), dtype=np.uint8)
    y = both(Q2_K, np.concatenate([scales, qs, f16b(1.0), f16b(0.0)]))
    e = np.arange(256)
    n, j, l = e // 128, (e % 128) // 32, e % 32
    group = 8 * n + 2 * j + (l >= 16)
    assert np.array_equal(y, group * np.array([1, 2, 3, 0])[j].astype(np.float64))
    # mins: high nibble, subtracted with dmin
    y = both(Q2_K, np.concatenate([(scales << 4).astype(np.uint8), np.zeros(64, np.uint8), f16b(1.0), f16b(0.5)]))
    assert np.array_equal(y, -0.5 * group)
    # distinct bytes: element e of a half reads byte 32n + l
    qs = np.arange(64, dtype=np.uint8)
    y = both(Q2_K, np.concatenate([np.full(16, 1, np.uint8), qs, f16b(1.0), f16b(0.0)]))
    assert np.array_equal(y, ((32 * n + l) >> (2 * j)) & 3)


def test_q5_k_fifth_bit_and_layout():
    # scales all 1, mins 0 (first eight packed bytes 1 / 0, last four 0x01): y = q
    scales = np.array([1, 1, 1, 1, 0, 0, 0, 0, 1, 1, 1, 1], dtype=np.uint8)
    qs = (np.arange(128) % 16).astype(np.uint8) | (((np.arange(128) + 5) % 16).astype(np.uint8) << 4)
    e = np.arange(256)
    c, r = e // 64, e % 64
    for sub in range(8):
        qh = np.full(32, 1 << sub, dtype=np.uint8)
        y = both(Q5_K, np.concatenate([f16b(1.0), f16b(0.0), scales, qh, qs]))
        byte = qs[32 * c + r % 32]
        nib = np.where(r < 32, byte & 0x0F, byte >> 4)
        want = nib + 16.0 * ((2 * c + (r >= 32)) == sub)  # bit `sub` of qh[l] belongs to sub-block `sub`
        assert np.array_equal(y, want), sub
    # a single qh byte: position l = r % 32
    qh = np.zeros(32, dtype=np.uint8)
    qh[7] = 0xFF
    y = both(Q5_K, np.concatenate([f16b(1.0), f16b(0.0), scales, qh, np.zeros(128, np.uint8)]))
    assert np.array_equal(np.nonzero(y)[0], np.arange(8) * 32 + 7)
    # 6-bit scales and mins use the Q4_K packing
    sc = np.array([[1, 2, 3, 4, 33, 34, 35, 63]], dtype=np.uint8)
    mn = np.array([[5, 6, 7, 8, 40, 41, 42, 60]], dtype=np.uint8)
    y = both(Q5_K, np.concatenate([f16b(2.0), f16b(1.0), synth.pack_q4k_scales(sc, mn)[0], np.zeros(32, np.uint8),
                                   np.full(128, 0x11, np.uint8)]))
    assert np.array_equal(y.reshape(8, 32)[:, 0], 2.0 * sc[0] * 1.0 - 1.0 * mn[0])


def _q3k_block(scales6, hmask, qs, d):
    """Pack sixteen 6-bit scale codes the way ggml stores them in twelve bytes."""
    s = np.zeros(12, dtype=np.uint8)
    for i, v in enumerate(scales6):
        if i < 8:
            s[i] |= v & 15
        else:
            s[i - 8] |= (v & 15) << 4
        s[8 + i % 4] |= (v >> 4) << (2 * (i // 4))
    return np.concatenate([hmask, qs, s, f16b(d)]).astype(np.uint8)


def test_q3_k_scales_high_bit_and_layout():
    e = np.arange(256)
    n, j, l = e // 128, (e % 128) // 32, e % 32
    group = 8 * n + 2 * j + (l >= 16)
    # every scale code distinct and above 32 (so both the low nibble and the two high bits matter); q = 1 with the
    # high-bit mask all set: y = d * (code - 32)
    codes = np.array([33, 47, 48, 63, 34, 50, 35, 62, 36, 44, 49, 61, 37, 40, 52, 60])
    y = both(Q3_K, _q3k_block(codes, np.full(32, 0xFF, np.uint8), np.full(64, 0x55, np.uint8), 0.5))
    assert np.array_equal(y, 0.5 * (codes[group] - 32))
    # codes below 32 are negative scales
    low = np.arange(16)
    y = both(Q3_K, _q3k_block(low, np.full(32, 0xFF, np.uint8), np.full(64, 0x55, np.uint8), 1.0))
    assert np.array_equal(y, (low[group] - 32.0))
    # a cleared mask bit subtracts 4: bit (4n + j) of hmask[l]
    for bit in range(8):
        y = both(Q3_K, _q3k_block(np.full(16, 33), np.full(32, 1 << bit, np.uint8), np.full(64, 0xFF, np.uint8), 1.0))
        assert np.array_equal(y, np.where(4 * n + j == bit, 3.0, -1.0)), bit
    hm = np.zeros(32, np.uint8)
    hm[9] = 0xFF
    y = both(Q3_K, _q3k_block(np.full(16, 33), hm, np.zeros(64, np.uint8), 1.0))
    assert np.array_equal(np.nonzero(y == 0.0)[0], np.arange(8) * 32 + 9)
    # distinct quant bytes: element reads byte 32n + l, bit pair j
    qs = (np.arange(64) * 7 % 256).astype(np.uint8)
    y = both(Q3_K, _q3k_block(np.full(16, 33), np.full(32, 0xFF, np.uint8), qs, 1.0))
    assert np.array_equal(y, (qs[32 * n + l] >> (2 * j)) & 3)


def test_q8_k_float_scale_and_ignored_sums():
    qs = np.arange(-128, 128, dtype=np.int8)
    d = np.array([0.1], dtype=np.float32)  # not representable in fp16: the scale really is a float32
    blk = np.concatenate([d.view(np.uint8), qs.view(np.uint8), np.zeros(32, np.uint8)])
    y = both(Q8_K, blk)
    assert np.array_equal(y, (d[0].astype(np.float64) * qs).astype(np.float32))
    blk[260:292] = 0xFF  # the trailing block sums do not change the values
    assert np.array_equal(both(Q8_K, blk), y)


def test_iq4_table_and_element_order():
    qs = np.array([j | ((15 - j) << 4) for j in range(16)], dtype=np.uint8)
    y = both(IQ4_NL, np.concatenate([f16b(2.0), qs]))
    assert np.array_equal(y[:16], 2.0 * IQ4)         # low nibbles first: the table in order
    assert np.array_equal(y[16:], 2.0 * IQ4[::-1])   # then high nibbles
    assert np.all(np.diff(IQ4) > 0) and IQ4.sum() == -94.0  # the published table: increasing, known checksum


def test_iq4_xs_scales_and_layout():
    # sub-block ib gets 6-bit code ls(ib): low nibble from scales_l, high two bits from scales_h
    codes = np.array([33, 47, 0, 63, 32, 16, 50, 31])
    sl = np.zeros(4, np.uint8)
    sh = 0
    for ib, v in enumerate(codes):
        sl[ib // 2] |= (v & 15) << (4 * (ib % 2))
        sh |= (v >> 4) << (2 * ib)
    qs = np.tile(np.array([j | ((15 - j) << 4) for j in range(16)], dtype=np.uint8), 8)
    blk = np.concatenate([f16b(0.25), np.array([sh & 0xFF, sh >> 8], np.uint8), sl, qs])
    y = both(IQ4_XS, blk).reshape(8, 32)
    for ib in range(8):
        assert np.array_equal(y[ib, :16], 0.25 * (codes[ib] - 32) * IQ4), ib
        assert np.array_equal(y[ib, 16:], 0.25 * (codes[ib] - 32) * IQ4[::-1]), ib
    # distinct bytes: sub-block ib reads qs[16 ib .. 16 ib + 15]
    qs = np.arange(128, dtype=np.uint8)
    blk = np.concatenate([f16b(1.0), np.array([0, 0], np.uint8), np.full(4, 0x11, np.uint8), qs])
    y = both(IQ4_XS, blk).reshape(8, 32)
    for ib in range(8):
        b = qs[16 * ib:16 * ib + 16]
        assert np.array_equal(y[ib], -31.0 * np.concatenate([IQ4[b & 15], IQ4[b >> 4]])), ib


def test_dense_types():
    v = np.array([0.0, -0.0, 1.0, -2.5, 65504.0, 6.1e-5, 5.96e-8], dtype=np.float32)
    assert np.array_equal(both(F16, v.astype(np.float16).view(np.uint8)), v.astype(np.float16).astype(np.float32))
    assert np.array_equal(both(BF16, synth.f32_to_bf16_bits(v).view(np.uint8)),
                          (synth.f32_to_bf16_bits(v).astype(np.uint32) << 16).view(np.float32))
    assert np.array_equal(both(F32, v.view(np.uint8)), v)


@pytest.mark.parametrize("qtype,name", MORE)
def test_matvec_reduces_to_dense(qtype, name):
    be, _ = synth.BLOCK[qtype]
    n, k = 5, 512
    raw = synth.weight(qtype, n, k, seed=qtype)
    x = synth.activation_f32(k, seed=1)
    w = oracle_c.dequant(qtype, raw).reshape(n, k).astype(np.float64)
    want = (w @ x.astype(np.float64)).astype(np.float32)
    assert np.array_equal(oracle_c.matvec_q(qtype, raw, n, k, x), want) or np.allclose(
        oracle_c.matvec_q(qtype, raw, n, k, x), want, rtol=1e-6)
    assert np.allclose(oracle_np.matvec_q(qtype, raw, n, k, x), want, rtol=1e-6)


def _trits5(v):
    return [(v // 3 ** (4 - n)) % 3 for n in range(5)]


def test_tq1_0_trit_packing_identity():
    """A byte stores five trits as ceil(v * 256 / 243): every one of the 243 values must come back, most
    significant trit first, through both oracles; the fourth-trit bytes of qh hold four trits and a zero."""
    d = f16b(0.5)
    for base in range(0, 243, 48):
        vals = [(base + i) % 243 for i in range(48)]
        qs = np.array([(v * 256 + 242) // 243 for v in vals], dtype=np.uint8)
        qh = np.array([(3 * v4 * 256 + 242) // 243 for v4 in (base % 81, 80, 0, 41)], dtype=np.uint8)
        y = both(TQ1_0, np.concatenate([qs, qh, d]))
        for n in range(5):
            want = np.array([_trits5(v)[n] - 1 for v in vals]) * 0.5
            assert np.array_equal(y[32 * n:32 * n + 32], want[:32]), (base, n)           # bytes 0..31: 32 n + m
            assert np.array_equal(y[160 + 16 * n:176 + 16 * n], want[32:]), (base, n)    # bytes 32..47: 160 + 16 n + m
        for n in range(4):
            want = np.array([_trits5(3 * v4)[n] - 1 for v4 in (base % 81, 80, 0, 41)]) * 0.5
            assert np.array_equal(y[240 + 4 * n:244 + 4 * n], want), (base, n)           # qh: 240 + 4 n + j


def test_tq2_0_element_order():
    # byte 32 g + m holds elements 128 g + 32 l + m in bit pairs l = 0..3
    qs = np.zeros(64, np.uint8)
    want = np.zeros(256)
    rng = np.random.default_rng(7)
    for g in range(2):
        for m in range(32):
            t = rng.integers(0, 3, size=4)
            qs[32 * g + m] = t[0] | (t[1] << 2) | (t[2] << 4) | (t[3] << 6)
            for l in range(4):
                want[128 * g + 32 * l + m] = (t[l] - 1) * -0.25
    y = both(TQ2_0, np.concatenate([qs, f16b(-0.25)]))
    assert np.array_equal(y, want.astype(np.float32))
    # all fields 1 -> zeros carrying the sign of d; all fields 2 -> +d; all 0 -> -d
    for fill, val in ((0x55, 0.0), (0xAA, -0.25), (0x00, 0.25)):
        y = both(TQ2_0, np.concatenate([np.full(64, fill, np.uint8), f16b(-0.25)]))
        assert np.all(y == val)
