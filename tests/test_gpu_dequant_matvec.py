"""GPU parity: dequantization (bit-exact) and batch-1 matvec (rel. error <= 1e-3) through the C ABI vs the CPU oracle."""
import os

import numpy as np
import pytest

from oracle import oracle_c, oracle_np
from skainet_amd import runtime, synth

pytestmark = pytest.mark.gpu

Q8_0, Q4_K, Q6_K = 8, 12, 14
TOL = 1e-3  # max_i |a_i - r_i| / max(|r_i|, 1e-3 * max|r|) against the fp64-accumulated oracle


@pytest.mark.parametrize("qtype,name", [(Q8_0, "q8_0"), (Q4_K, "q4_k"), (Q6_K, "q6_k")])
def test_dequant_golden_blocks_bit_exact(hip, golden_dir, qtype, name):
    blocks = np.load(os.path.join(golden_dir, "quant_blocks.npz"))
    got = hip.dequant_host(qtype, blocks[f"{name}_raw"])
    assert np.array_equal(got.view(np.uint32), blocks[f"{name}_f32_bits"])


@pytest.mark.parametrize("qtype", [Q8_0, Q4_K, Q6_K])
def test_dequant_bit_exact_vs_oracle(hip, qtype):
    be, bb = synth.BLOCK[qtype]
    raw = synth.weight(qtype, 512, 4096, seed=100 + qtype)
    got = hip.dequant_host(qtype, raw)
    want = oracle_c.dequant(qtype, raw)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # arbitrary bytes (random f16 scales incl. subnormals and negatives; inf / nan scales excluded)
    rng = np.random.default_rng(7 + qtype)
    rnd = rng.integers(0, 256, size=(4096, bb), dtype=np.uint8)
    for p in {Q8_0: [1], Q4_K: [1, 3], Q6_K: [209]}[qtype]:
        rnd[:, p] &= 0xFB
    got = hip.dequant_host(qtype, rnd.reshape(-1))
    want = oracle_c.dequant(qtype, rnd.reshape(-1))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_dequant_full_size_checksum(hip):
    # full benchmark tensor (Q4_K 4096 x 11008): compared through a 64-bit sum of the output words
    raw = synth.weight(Q4_K, 4096, 11008, seed=42)
    got = hip.dequant_host(Q4_K, raw)
    want = oracle_c.dequant(Q4_K, raw)
    assert int(got.view(np.uint32).astype(np.uint64).sum()) == int(want.view(np.uint32).astype(np.uint64).sum())
    assert np.array_equal(got[:: 4099].view(np.uint32), want[:: 4099].view(np.uint32))


def test_dequant_errors(hip):
    buf = hip.alloc(1024)
    with pytest.raises(runtime.SknError) as e:
        hip.dequant(16, buf, 256, buf)  # IQ2_XXS: in the size table, not computed with
    assert e.value.code == runtime.ERR_TYPE
    with pytest.raises(runtime.SknError) as e:
        hip.dequant(Q4_K, buf, 100, buf)
    assert e.value.code == runtime.ERR_SHAPE
    with pytest.raises(runtime.SknError) as e:
        hip.dequant(Q4_K, None, 256, buf)
    assert e.value.code == runtime.ERR_ARG
    hip.dequant(Q4_K, buf, 0, buf)  # empty input is a no-op


MATVEC_CASES = [
    (Q8_0, 4096, 4096),
    (Q4_K, 4096, 4096),
    (Q4_K, 11008, 4096),
    (Q4_K, 4096, 11008),
    (Q6_K, 4096, 4096),
    # ragged: rows not a multiple of the workgroup, K from one superblock up to a non-power-of-two count
    (Q4_K, 37, 256),
    (Q4_K, 5, 2304),
    (Q4_K, 100, 13 * 256),
    (Q4_K, 3, 57 * 256),
    (Q8_0, 33, 96),
    (Q8_0, 7, 32 * 131),
    # Q8_0 rows that are whole block pairs: one lane step partly filled, several steps, the largest unrolled
    # size, and one past it (general kernel)
    (Q8_0, 3, 64),
    (Q8_0, 5, 64 * 70),
    (Q8_0, 17, 8192),
    (Q8_0, 2, 12800),
    (Q8_0, 9, 16384),
    (Q8_0, 4, 16384 + 64),
    (Q6_K, 19, 768),
    (Q6_K, 5, 256),
    (Q6_K, 33, 256 * 17),
    (Q6_K, 3, 256 * 50),
    (Q6_K, 2, 16384),
    (Q6_K, 2, 16384 + 256),  # past the unrolled sizes: general kernel
    (Q6_K, 1000, 4096),
]


@pytest.mark.parametrize("qtype,n,k", MATVEC_CASES)
def test_matvec_vs_oracle(hip, qtype, n, k):
    raw = synth.weight(qtype, n, k, seed=n * 7 + k)
    x = synth.activation_f32(k, seed=k + 1)
    got = hip.matvec_q_host(qtype, raw, n, k, x)
    want = oracle_c.matvec_q(qtype, raw, n, k, x)
    err = oracle_np.rel_err(got, want)
    assert err <= TOL, f"rel err {err}"


@pytest.mark.parametrize("nb", [16, 17, 32, 33, 48, 49, 64, 65, 144])
def test_matvec_q4k_step_boundaries(hip, nb):
    """Q4_K rows of exactly 1, 2, 3 and 4 sixteen-superblock steps and one superblock past each (the unrolled
    kernels end at 64; 144 superblocks is the longest row whose staging fits the LDS), with row counts around the
    rows a workgroup takes."""
    k = 256 * nb
    for n in (1, 7, 8, 9, 15, 16, 17, 31):
        raw = synth.weight(Q4_K, n, k, seed=nb * 100 + n)
        x = synth.activation_f32(k, seed=nb + n)
        got = hip.matvec_q_host(Q4_K, raw, n, k, x)
        want = oracle_c.matvec_q(Q4_K, raw, n, k, x)
        assert oracle_np.rel_err(got, want) <= TOL, (nb, n)


def test_matvec_extreme_activations(hip):
    """fp32 activations towards the ends of the range: zeros, 1e-28 (the Q4_K kernel works in units of 2^-24 and
    flushes what is smaller than about 2^-100), 1e30, one huge element among small ones."""
    n, k = 24, 4096
    rng = np.random.default_rng(77)
    for qtype in (Q8_0, Q4_K, Q6_K):
        raw = synth.weight(qtype, n, k, seed=qtype)
        for kind in range(5):
            x = rng.standard_normal(k).astype(np.float32)
            if kind == 0:
                x[:] = 0.0
            elif kind == 1:
                x *= 1e-28
            elif kind == 2:
                x *= 1e30
            elif kind == 3:
                x *= 1e-6
                x[1234] = 3.0e8
            else:
                x[::2] = 0.0
            got = hip.matvec_q_host(qtype, raw, n, k, x)
            want = oracle_c.matvec_q(qtype, raw, n, k, x)
            assert np.all(np.isfinite(got)), (qtype, kind)
            if kind == 0:
                assert np.all(got == 0.0)
            else:
                assert oracle_np.rel_err(got, want) <= TOL, (qtype, kind)


@pytest.mark.parametrize("qtype", [Q8_0, Q4_K, Q6_K])
def test_matvec_one_hot_and_linearity(hip, qtype):
    n, k = 64, 2048
    raw = synth.weight(qtype, n, k, seed=5)
    w = oracle_c.dequant(qtype, raw).reshape(n, k)
    for col in (0, 31, 32, 255, 256, 1029, k - 1):
        e = np.zeros(k, dtype=np.float32)
        e[col] = 1.0
        got = hip.matvec_q_host(qtype, raw, n, k, e)
        assert np.allclose(got, w[:, col], rtol=1e-6, atol=1e-7), col
    x1 = synth.activation_f32(k, seed=1)
    x2 = synth.activation_f32(k, seed=2)
    y1 = hip.matvec_q_host(qtype, raw, n, k, x1).astype(np.float64)
    y2 = hip.matvec_q_host(qtype, raw, n, k, x2).astype(np.float64)
    y12 = hip.matvec_q_host(qtype, raw, n, k, 2.0 * x1 - x2).astype(np.float64)
    assert oracle_np.rel_err(y12, 2.0 * y1 - y2) <= TOL


def test_matvec_errors_and_empty(hip):
    buf = hip.alloc(4096)
    with pytest.raises(runtime.SknError) as e:
        hip.matvec_q(Q4_K, buf, 4, 200, buf, buf)
    assert e.value.code == runtime.ERR_SHAPE
    assert "is not a multiple of block size (256)" in e.value.message
    with pytest.raises(runtime.SknError) as e:
        hip.matvec_q(16, buf, 4, 256, buf, buf)
    assert e.value.code == runtime.ERR_TYPE
    with pytest.raises(runtime.SknError) as e:
        hip.matvec_q(Q4_K, buf, 4, 256, None, buf)
    assert e.value.code == runtime.ERR_ARG
    hip.matvec_q(Q4_K, buf, 0, 256, buf, buf)
    y = hip.to_device(np.ones(4, dtype=np.float32))
    hip.matvec_q(Q4_K, buf, 4, 0, buf, y)  # k = 0: the empty sum
    assert np.all(y.download(np.float32, 4) == 0.0)


def test_measuring_build_of_the_q4k_matvec(hip):
    """skn_test_matvec_q4k_stamps (what `bench.py --mode timeline` runs): the same result as skn_matvec_q bit for bit, and
    per wavefront seven clock readings in program order plus its hardware ids."""
    n, k = 72, 11008
    raw = synth.weight(Q4_K, n, k, seed=91)
    x = synth.activation_f32(k, seed=92)
    w, xd, y, stamps = hip.to_device(raw), hip.to_device(x), hip.alloc(4 * n), hip.alloc(64 * n)
    hip.test_matvec_q4k_stamps(w, n, k, xd, y, stamps)
    got = y.download(np.float32, n)
    assert np.array_equal(got.view(np.uint32), hip.matvec_q_host(Q4_K, raw, n, k, x).view(np.uint32))
    t = stamps.download(np.uint64, 8 * n).reshape(n, 8)
    assert np.all(t[:, 0] > 0) and np.all(np.diff(t[:, :7].astype(np.int64), axis=1) >= 0)
    assert np.all((t[:, 7] >> np.uint64(32)) < 8)  # XCC_ID
    with pytest.raises(runtime.SknError, match="multiple of 256 in"):
        hip.test_matvec_q4k_stamps(w, n, 4096, xd, y, stamps)
    with pytest.raises(runtime.SknError, match="multiple of 8"):  # (stamps are written per wavefront of whole workgroups)
        hip.test_matvec_q4k_stamps(w, n - 3, k, xd, y, stamps)
    for b in (w, xd, y, stamps):
        b.free()


@pytest.mark.parametrize("n,k", [(4096, 11008), (70, 4096), (64, 8192), (33, 256)])
@pytest.mark.parametrize("split,rows", [(1, 1), (1, 2), (2, 1), (2, 2)])
def test_q4k_matvec_with_k_split_across_workgroups(hip, n, k, split, rows):
    """Option q4k.split: a workgroup takes one step of sixteen superblocks of its rows; partials merged behind a ticket
    (1: the sum runs in slice order, so two calls give the same bits) or by atomic adds into a zeroed y (2).  Same
    answer as the oracle at the operation's bound, at the headline shape, with a ragged last row group, with two and
    one slices; the ticket counters are back at zero after every call (a second call on another weight is right too)."""
    raw = synth.weight(synth.Q4_K, n, k, seed=300 + n)
    raw2 = synth.weight(synth.Q4_K, n, k, seed=301 + n)
    x = synth.activation_f32(k, seed=302)
    w, w2, xd, y = hip.to_device(raw), hip.to_device(raw2), hip.to_device(x), hip.alloc(4 * n)
    hip.set_option("q4k.split", split)
    hip.set_option("q4k.rows", rows)
    try:
        hip.matvec_q(synth.Q4_K, w, n, k, xd, y)
        first = y.download(np.float32, n)
        assert oracle_np.rel_err(first, oracle_c.matvec_q(synth.Q4_K, raw, n, k, x)) <= 1e-3
        hip.matvec_q(synth.Q4_K, w2, n, k, xd, y)
        assert oracle_np.rel_err(y.download(np.float32, n), oracle_c.matvec_q(synth.Q4_K, raw2, n, k, x)) <= 1e-3
        hip.matvec_q(synth.Q4_K, w, n, k, xd, y)
        again = y.download(np.float32, n)
        if split == 1:
            assert np.array_equal(first.view(np.uint32), again.view(np.uint32))
        else:
            assert oracle_np.rel_err(again, first) <= 1e-4  # (the order of the atomic additions moves the last bit)
    finally:
        hip.set_option("q4k.split", 0)
        hip.set_option("q4k.rows", 0)
    for b in (w, w2, xd, y):
        b.free()
