"""GPU parity for the further ggml formats (Q4_0, Q4_1, Q5_0, Q5_1, Q2_K, Q3_K, Q5_K, Q8_K, IQ4_NL, IQ4_XS, TQ1_0,
TQ2_0, F16, BF16, F32) through the C ABI:
dequantization bit for bit against the CPU oracle, matvec and GEMM within the 1e-3 criterion."""
import numpy as np
import pytest

from oracle import oracle_c, oracle_np
from skainet_amd import runtime, synth

pytestmark = pytest.mark.gpu
TOL = 1e-3
MORE = [(2, "q4_0"), (3, "q4_1"), (6, "q5_0"), (7, "q5_1"), (10, "q2_k"), (13, "q5_k"), (11, "q3_k"), (15, "q8_k"),
        (20, "iq4_nl"), (23, "iq4_xs"), (34, "tq1_0"), (35, "tq2_0"), (1, "f16"), (30, "bf16"), (0, "f32")]


@pytest.mark.parametrize("qtype,name", MORE)
def test_dequant_bit_exact(hip, qtype, name):
    be, bb = synth.BLOCK[qtype]
    n, k = 37, 1536 if be > 1 else 1001
    raw = synth.weight(qtype, n, k, seed=qtype + 50)
    want = oracle_c.dequant(qtype, raw)
    out = hip.alloc(4 * n * k)
    hip.dequant(qtype, hip.to_device(raw), n * k, out)
    got = out.download(np.float32, n * k)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("qtype,name", [t for t in MORE if t[0] not in (0, 1, 30)])
def test_dequant_random_bytes_bit_exact(hip, qtype, name):
    """Uniform random payload bytes (all scale / min / bit patterns), finite fp16 fields."""
    be, bb = synth.BLOCK[qtype]
    raw = np.random.default_rng(qtype).integers(0, 256, size=4096 * bb, dtype=np.uint8)
    for off in {2: (0,), 3: (0, 2), 6: (0,), 7: (0, 2), 10: (80, 82), 13: (0, 2), 11: (108,), 15: (2,), 20: (0,),
                23: (0,), 34: (52,), 35: (64,)}[qtype]:
        raw.reshape(-1, bb)[:, off + 1] &= 0x7B  # (Q8_K: the top byte of its float32 scale)
    want = oracle_c.dequant(qtype, raw)
    out = hip.alloc(4 * want.size)
    hip.dequant(qtype, hip.to_device(raw), want.size, out)
    got = out.download(np.float32, want.size)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("qtype,name", [t for t in MORE if t[0] not in (0, 1, 30)])
def test_dequant_golden_blocks(hip, golden_dir, qtype, name):
    import os
    g = np.load(os.path.join(golden_dir, "quant_blocks_more.npz"))
    raw, want = g[f"{name}_raw"], g[f"{name}_f32_bits"]
    out = hip.alloc(4 * want.size)
    hip.dequant(qtype, hip.to_device(raw), want.size, out)
    assert np.array_equal(out.download(np.float32, want.size).view(np.uint32), want)


@pytest.mark.parametrize("qtype,name", MORE)
@pytest.mark.parametrize("n,k", [(64, 4096), (5, 768), (1, 256)])
def test_matvec_vs_oracle(hip, qtype, name, n, k):
    raw = synth.weight(qtype, n, k, seed=n + k + qtype)
    x = synth.activation_f32(k, seed=k)
    got = hip.matvec_q_host(qtype, raw, n, k, x)
    want = oracle_c.matvec_q(qtype, raw, n, k, x)
    assert oracle_np.rel_err(got, want) <= TOL


STAGED = [(2, "q4_0"), (3, "q4_1"), (6, "q5_0"), (7, "q5_1"), (20, "iq4_nl"), (10, "q2_k"), (13, "q5_k"), (15, "q8_k"), (23, "iq4_xs"),
          (11, "q3_k")]


@pytest.mark.parametrize("qtype,name", STAGED)
@pytest.mark.parametrize("n,k", [(7, 11008), (4, 16384), (9, 2048), (3, 256)])
def test_matvec_staged_and_plain_kernels(hip, qtype, name, n, k):
    """The formats whose rows pass through LDS: several chunks per row with a short last one (k = 11008), the
    longest row, fewer rows than a workgroup takes -- every kernel the option selects (0: direct reads, 2: row
    staged in LDS, 1: the default, which for Q5_K, the small-block formats and IQ4_XS is the kernel on the Q4_K lane
    map and for Q2_K / Q3_K the one on the Q6_K lane map) against the oracle and against each other."""
    raw = synth.weight(qtype, n, k, seed=3 * n + k + qtype)
    x = synth.activation_f32(k, seed=k + 1)
    want = oracle_c.matvec_q(qtype, raw, n, k, x)
    got = {}
    try:
        for stage in (0, 1, 2):
            hip.set_option("matvec.stage", stage)
            got[stage] = hip.matvec_q_host(qtype, raw, n, k, x)
            assert oracle_np.rel_err(got[stage], want) <= TOL
    finally:
        hip.set_option("matvec.stage", 1)
    for stage in (1, 2):  # (fp32 sums in a different order)
        assert np.abs(got[stage] - got[0]).max() <= 1e-5 * np.abs(want).max()


@pytest.mark.parametrize("qtype,name", [(13, "q5_k"), (2, "q4_0"), (3, "q4_1"), (6, "q5_0"), (7, "q5_1"), (20, "iq4_nl"),
                                        (23, "iq4_xs"), (10, "q2_k"), (11, "q3_k"), (15, "q8_k"), (35, "tq2_0"), (34, "tq1_0")])
@pytest.mark.parametrize("n,k", [(33, 256), (16, 4096), (17, 8192), (9, 8448), (5, 12288), (3, 16384), (2, 36864), (1, 37120)])
def test_lane_map_matvec_every_step_count(hip, qtype, name, n, k):
    """The formats on the Q4_K kernel's lane map: rows of one to four unrolled steps (16 superblocks, or 16 groups of
    eight small blocks, each), a partial last step, the rolled loop beyond four steps, the longest row the kernel
    takes (144 superblocks) and one past it (direct kernel).  Q2_K and Q3_K (the Q6_K kernel's lane map) and Q8_K: one
    to four steps, then the kernels for longer rows; TQ2_0 likewise (the packing of Q2_K's quants) and TQ1_0 (a lane map
    of its own)."""
    raw = synth.weight(qtype, n, k, seed=n + k)
    x = synth.activation_f32(k, seed=k + 3)
    got = hip.matvec_q_host(qtype, raw, n, k, x)
    assert oracle_np.rel_err(got, oracle_c.matvec_q(qtype, raw, n, k, x)) <= TOL


@pytest.mark.parametrize("qtype,name,bb", [(2, "q4_0", 18), (3, "q4_1", 20), (6, "q5_0", 22), (7, "q5_1", 24), (20, "iq4_nl", 18)])
def test_small_block_matvec_field_positions(hip, qtype, name, bb):
    """Q4_0 / Q4_1 / Q5_0 / Q5_1 / IQ4_NL with one block of every pair zeroed, with only low or only high nibbles set and
    (the five-bit formats) with only one half of the fifth bits set: the realigned first block, the aligned second
    one and every bit plane against the oracle on their own."""
    n, k = 8, 2048
    raw = synth.weight(qtype, n, k, seed=31).reshape(n, k // 32, bb).copy()
    x = synth.activation_f32(k, seed=32)
    variants = []
    for keep in (0, 1):
        v = raw.copy()
        v[:, 1 - keep::2, :] = 0
        variants.append(v)
    for mask in (0x0F, 0xF0):
        v = raw.copy()
        v[:, :, bb - 16:] &= mask
        variants.append(v)
    if bb >= 22:  # the four bytes before the nibbles: fifth bits of elements 0..15 (first two), 16..31 (last two)
        for lo, hi in ((bb - 20, bb - 18), (bb - 18, bb - 16)):
            v = raw.copy()
            v[:, :, bb - 16:] = 0
            v[:, :, lo:hi] = 0
            variants.append(v)
    for v in variants:
        got = hip.matvec_q_host(qtype, v.reshape(n, -1), n, k, x)
        assert oracle_np.rel_err(got, oracle_c.matvec_q(qtype, v.reshape(n, -1), n, k, x)) <= TOL


def test_q5k_matvec_fifth_bits_alone(hip):
    """Quants whose nibbles are all zero and whose fifth bits are random, and the reverse: each bit plane of the
    kernel against the oracle separately (a misplaced qh bit or sub-block shift shows at full scale)."""
    n, k = 8, 4096
    rng = np.random.default_rng(5)
    raw = synth.weight(13, n, k, seed=21).reshape(n, k // 256, 176).copy()
    x = synth.activation_f32(k, seed=22)
    only_bits = raw.copy()
    only_bits[:, :, 48:] = 0
    only_bits[:, :, 16:48] = rng.integers(0, 256, size=(n, k // 256, 32), dtype=np.uint8)
    only_nibbles = raw.copy()
    only_nibbles[:, :, 16:48] = 0
    for blocks in (only_bits, only_nibbles):
        got = hip.matvec_q_host(13, blocks.reshape(n, -1), n, k, x)
        assert oracle_np.rel_err(got, oracle_c.matvec_q(13, blocks.reshape(n, -1), n, k, x)) <= TOL


@pytest.mark.parametrize("qtype,name", [(3, "q4_1"), (10, "q2_k")])
def test_matvec_rows_not_16_byte_aligned(hip, qtype, name):
    """Rows whose byte length is not a multiple of 16 (three Q4_1 blocks, one Q2_K block) and a weight pointer off
    the 16-byte grid take the kernel that reads global memory directly."""
    be, bb = synth.BLOCK[qtype]
    n, k = 6, 3 * be if qtype == 3 else be
    raw = synth.weight(qtype, n, k, seed=11)
    x = synth.activation_f32(k, seed=12)
    want = oracle_c.matvec_q(qtype, raw, n, k, x)
    assert oracle_np.rel_err(hip.matvec_q_host(qtype, raw, n, k, x), want) <= TOL
    # base pointer 4 bytes into an allocation
    n, k = 5, 16 * be
    raw = synth.weight(qtype, n, k, seed=13)
    x = synth.activation_f32(k, seed=14)
    buf = hip.alloc(raw.nbytes + 16)
    flat = np.concatenate([np.zeros(4, np.uint8), raw.reshape(-1)])
    buf.upload(flat)
    xd, yd = hip.to_device(x), hip.alloc(4 * n)
    hip.matvec_q(qtype, buf.ptr + 4, n, k, xd, yd)
    assert oracle_np.rel_err(yd.download(np.float32, n), oracle_c.matvec_q(qtype, raw, n, k, x)) <= TOL


def _against_oracle(hip, qtype, blocks, n, k, x):
    got = hip.matvec_q_host(qtype, blocks.reshape(n, -1), n, k, x)
    assert oracle_np.rel_err(got, oracle_c.matvec_q(qtype, blocks.reshape(n, -1), n, k, x)) <= TOL


def test_q2k_matvec_fields_alone(hip):
    """Q2_K (scales[16] @0, qs[64] @16, d @80, dmin @82) on the lane-map kernel, one field at a time: scales without
    minimums and the reverse, each bit pair of qs alone, the bytes of either half of a run alone, one half of the
    superblock alone -- a wrong scale index, shift or run sum shows at full scale."""
    n, k = 16, 4096
    raw = synth.weight(10, n, k, seed=41).reshape(n, k // 256, 84).copy()
    x = synth.activation_f32(k, seed=42)
    variants = []
    for mask in (0x0F, 0xF0):
        v = raw.copy()
        v[:, :, :16] &= mask
        variants.append(v)
    for j in range(4):
        v = raw.copy()
        v[:, :, 16:80] &= 3 << (2 * j)
        variants.append(v)
    for lo in (0, 16):  # bytes l = lo .. lo + 15 of both halves
        v = raw.copy()
        keep = np.zeros(64, bool)
        keep[lo:lo + 16] = keep[32 + lo:48 + lo] = True
        v[:, :, 16:80][:, :, ~keep] = 0
        v[:, :, :16] &= 0x0F  # (no minimums: the zeroed quants contribute nothing)
        variants.append(v)
    for half in (0, 1):
        v = raw.copy()
        v[:, :, 16 + 32 * (1 - half):48 + 32 * (1 - half)] = 0
        v[:, :, 8 * (1 - half):8 + 8 * (1 - half)] = 0
        variants.append(v)
    for v in variants:
        _against_oracle(hip, 10, v, n, k, x)


def test_q3k_matvec_fields_alone(hip):
    """Q3_K (hmask[32] @0, qs[64] @32, scales[12] @96, d @108): third bits all set (quants 0..3) or all clear (-4..-1)
    or alone over zero low bits, each bit pair alone, each of the eight bit planes of hmask alone, the three parts of
    the packed scales alone (low nibbles of bytes 0..7 = scales 0..7, high nibbles = 8..15, bytes 8..11 = the upper
    two bits), one half alone."""
    n, k = 16, 4096
    rng = np.random.default_rng(6)
    raw = synth.weight(11, n, k, seed=43).reshape(n, k // 256, 110).copy()
    x = synth.activation_f32(k, seed=44)
    variants = []
    for fill in (0xFF, 0x00):
        v = raw.copy()
        v[:, :, :32] = fill
        variants.append(v)
    v = raw.copy()
    v[:, :, 32:96] = 0
    variants.append(v)
    for j in range(4):
        v = raw.copy()
        v[:, :, 32:96] &= 3 << (2 * j)
        variants.append(v)
    for bit in range(8):
        v = raw.copy()
        v[:, :, :32] = (rng.integers(0, 2, size=(n, k // 256, 32), dtype=np.uint8) << bit) | (0xFF ^ (1 << bit))
        v[:, :, 32:96] = 0  # quants: -4 where the plane's bit is clear, 0 elsewhere
        variants.append(v)
    for part in range(3):
        v = raw.copy()
        if part == 0:
            v[:, :, 96:104] &= 0x0F
            v[:, :, 104:108] = 0xAA  # upper bits 2: scales 32 + low nibble - 32
        elif part == 1:
            v[:, :, 96:104] &= 0xF0
            v[:, :, 104:108] = 0xAA
        else:
            v[:, :, 96:104] = 0
        variants.append(v)
    for half in (0, 1):
        v = raw.copy()
        v[:, :, 32 + 32 * (1 - half):64 + 32 * (1 - half)] = 0
        v[:, :, :32] |= 0x0F << (4 * (1 - half))  # the zeroed half's quants are 0, not -4
        variants.append(v)
    for v in variants:
        _against_oracle(hip, 11, v, n, k, x)


def test_tq2_0_matvec_bit_pairs_alone(hip):
    """TQ2_0 (qs[64] @0, d @64; y = d (q - 1)) on the lane-map kernel: each bit pair alone, each half alone, all quants 2
    (y = d sum x) and all quants 1 (every weight zero)."""
    n, k = 16, 4096
    raw = synth.weight(35, n, k, seed=61).reshape(n, k // 256, 66).copy()
    x = synth.activation_f32(k, seed=62)
    variants = [raw]
    for j in range(4):
        v = raw.copy()
        v[:, :, :64] &= 3 << (2 * j)
        variants.append(v)
    for half in (0, 1):
        v = raw.copy()
        v[:, :, 32 * (1 - half):32 * (1 - half) + 32] = 0x55  # the other half: quants 1, weights 0
        variants.append(v)
    v = raw.copy()
    v[:, :, :64] = 0xAA
    variants.append(v)
    for v in variants:
        _against_oracle(hip, 35, v, n, k, x)
    # all quants 1: every weight is zero, and what is left of sum(q x) - sum(x) is rounding noise
    v = raw.copy()
    v[:, :, :64] = 0x55
    got = hip.matvec_q_host(35, v.reshape(n, -1), n, k, x)
    assert np.abs(got).max() <= 1e-5 * np.abs(x).sum() * 0.05


def test_tq1_0_matvec_regions_alone(hip):
    """TQ1_0 (qs[48] @0, qh[4] @48, d @52; five trits per byte, four per qh byte; y = d (t - 1)) on its lane-map kernel:
    each of the three regions of a block alone and each lane's bytes alone (every other byte 0x80: all its trits 1, its
    weights zero), all trits 2 (byte 255: y = d sum x), all trits 0 (byte 0: y = -d sum x), odd rows (2-byte aligned)."""
    n, k = 15, 4096 + 256
    raw = synth.weight(34, n, k, seed=71).reshape(n, k // 256, 54).copy()
    x = synth.activation_f32(k, seed=72)
    variants = [raw]
    for lo, hi in ((0, 32), (32, 48), (48, 52)):
        v = raw.copy()
        keep = np.zeros(52, bool)
        keep[lo:hi] = True
        v[:, :, :52][:, :, ~keep] = 0x80
        variants.append(v)
    for jj in range(4):
        v = raw.copy()
        keep = np.zeros(52, bool)
        keep[8 * jj:8 * jj + 8] = keep[32 + 4 * jj:36 + 4 * jj] = keep[48 + jj] = True
        v[:, :, :52][:, :, ~keep] = 0x80
        variants.append(v)
    for fill in (255, 0):
        v = raw.copy()
        v[:, :, :52] = fill
        variants.append(v)
    for v in variants:
        _against_oracle(hip, 34, v, n, k, x)
    # all trits 1: every weight is zero, and what is left of sum(t x) - sum(x) is rounding noise
    v = raw.copy()
    v[:, :, :52] = 0x80
    got = hip.matvec_q_host(34, v.reshape(n, -1), n, k, x)
    assert np.abs(got).max() <= 1e-5 * np.abs(x).sum() * 0.05


def test_q8k_matvec_ignores_the_block_sums(hip):
    """Q8_K (f32 d @0, int8 qs[256] @4, int16 sums @260) on the lane-map kernel: the stored sums of sixteen are not part
    of the values (random bytes there change nothing); each quarter of a superblock alone; the extreme quants."""
    n, k = 16, 4096
    rng = np.random.default_rng(9)
    raw = synth.weight(15, n, k, seed=51).reshape(n, k // 256, 292).copy()
    x = synth.activation_f32(k, seed=52)
    base = hip.matvec_q_host(15, raw.reshape(n, -1), n, k, x)
    _against_oracle(hip, 15, raw, n, k, x)
    v = raw.copy()
    v[:, :, 260:] = rng.integers(0, 256, size=(n, k // 256, 32), dtype=np.uint8)
    assert np.array_equal(hip.matvec_q_host(15, v.reshape(n, -1), n, k, x), base)
    for quarter in range(4):
        v = raw.copy()
        keep = np.zeros(256, bool)
        keep[64 * quarter:64 * quarter + 64] = True
        v[:, :, 4:260][:, :, ~keep] = 0
        _against_oracle(hip, 15, v, n, k, x)
    for fill in (0x80, 0x7F):  # -128 and 127 everywhere
        v = raw.copy()
        v[:, :, 4:260] = fill
        _against_oracle(hip, 15, v, n, k, x)


def test_iq4_xs_matvec_fields_alone(hip):
    """IQ4_XS (d @0, scales_h @2, scales_l[4] @4, qs[128] @8): the upper scale bits alone and the lower alone, low
    nibbles and high nibbles alone, each sub-block alone, and every table entry (all nibbles one index, scale 33 - 32)."""
    n, k = 16, 4096
    raw = synth.weight(23, n, k, seed=45).reshape(n, k // 256, 136).copy()
    x = synth.activation_f32(k, seed=46)
    variants = []
    v = raw.copy()
    v[:, :, 4:8] = 0
    variants.append(v)
    v = raw.copy()
    v[:, :, 2:4] = 0
    variants.append(v)
    for mask in (0x0F, 0xF0):
        v = raw.copy()
        v[:, :, 8:] &= mask
        v[:, :, 8:] |= 0x88 & ~mask  # index 8 of the table is the value 1, its smallest: the other nibbles nearly vanish
        variants.append(v)
    for ib in range(8):
        v = raw.copy()
        # scale 32 - 32 = 0 for every other sub-block: low bits 0, upper bits 2
        sl = np.zeros(4, np.uint8)
        sh = 0
        for o in range(8):
            val = 0x21 if o == ib else 0x20  # 33 or 32
            sl[o // 2] |= (val & 0xF) << (4 * (o % 2))
            sh |= (val >> 4) << (2 * o)
        v[:, :, 4:8] = sl
        v[:, :, 2] = sh & 0xFF
        v[:, :, 3] = sh >> 8
        variants.append(v)
    for v in variants:
        _against_oracle(hip, 23, v, n, k, x)
    k = 1024
    x = synth.activation_f32(k, seed=47)
    blocks = np.zeros((16, k // 256, 136), np.uint8)
    blocks[:, :, :2] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
    blocks[:, :, 2:4] = np.frombuffer(np.uint16(0xAAAA).tobytes(), np.uint8)  # upper bits 2 everywhere
    blocks[:, :, 4:8] = 0x11                                                   # lower bits 1: scale 33 - 32 = 1
    for i in range(16):
        blocks[i, :, 8:] = i | (i << 4)
    got = hip.matvec_q_host(23, blocks.reshape(16, -1), 16, k, x)
    want = oracle_c.matvec_q(23, blocks.reshape(16, -1), 16, k, x)
    table = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.float64)
    assert np.allclose(want, 0.5 * table * x.astype(np.float64).sum(), rtol=1e-5, atol=1e-4)
    assert oracle_np.rel_err(got, want) <= TOL


def test_iq4_nl_matvec_every_table_entry(hip):
    """IQ4_NL blocks whose nibbles are all one index, for each of the sixteen: the lookup of the lane-map kernel
    entry by entry (y = d * table[i] * sum(x))."""
    n, k = 16, 1024
    x = synth.activation_f32(k, seed=77)
    raw = np.zeros((n, k // 32, 18), np.uint8)
    raw[:, :, :2] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
    for i in range(16):
        raw[i, :, 2:] = i | (i << 4)
    got = hip.matvec_q_host(20, raw.reshape(n, -1), n, k, x)
    want = oracle_c.matvec_q(20, raw.reshape(n, -1), n, k, x)
    table = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.float64)
    assert np.allclose(want, 0.5 * table * x.astype(np.float64).sum(), rtol=1e-5, atol=1e-4)
    assert oracle_np.rel_err(got, want) <= TOL


def test_dense_matvec_odd_row_length(hip):
    for qtype in (0, 1, 30):
        n, k = 9, 333  # no block structure: any row length
        raw = synth.weight(qtype, n, k, seed=5)
        x = synth.activation_f32(k, seed=6)
        got = hip.matvec_q_host(qtype, raw, n, k, x)
        assert oracle_np.rel_err(got, oracle_c.matvec_q(qtype, raw, n, k, x)) <= TOL


@pytest.mark.parametrize("qtype,name", MORE)
def test_gemm_vs_oracle(hip, qtype, name):
    m, n, k = 48, 96, 1024
    raw = synth.weight(qtype, n, k, seed=qtype + 7)
    a = synth.activation_bf16((m, k), seed=8)
    got = hip.gemm_q_host(qtype, raw, n, k, a, m)
    want = oracle_c.gemm_q(qtype, raw, n, k, a, m)
    assert oracle_np.rel_err(got, want) <= TOL


def test_unknown_types_are_rejected(hip):
    buf = hip.alloc(4096)
    for qtype in (9, 16, 22, 4, 36):  # in the size table but not computed with / not in the table at all
        with pytest.raises(runtime.SknError) as e:
            hip.matvec_q(qtype, buf, 1, 256, buf, buf)
        assert e.value.code == runtime.ERR_TYPE
        with pytest.raises(runtime.SknError) as e:
            hip.dequant(qtype, buf, 256, buf)
        assert e.value.code == runtime.ERR_TYPE
