"""CPU: attention, KV shadow and decoder-glue oracles against closed forms and independent library routines."""
import numpy as np
import scipy.special

from oracle import oracle_c, oracle_np
from skainet_amd import synth


def test_attention_closed_forms():
    s, h, d, t = 2, 3, 16, 37
    q = np.random.default_rng(0).standard_normal((s, h, d)).astype(np.float32)
    k = synth.kv_f16((s, t, h, d), seed=1)
    v = synth.kv_f16((s, t, h, d), seed=2)
    # one token: the output is that token's V row exactly
    out = oracle_c.attn_decode(q, k, v, [1, 1], 0.25)
    assert np.array_equal(out, v[:, 0].view(np.float16).astype(np.float32))
    # identical keys: uniform weights, output is the mean of V
    ku = np.broadcast_to(k[:, :1], k.shape).copy()
    out = oracle_c.attn_decode(q, ku, v, [t, 20], 0.25)
    vf = v.view(np.float16).astype(np.float64)
    assert np.allclose(out[0], vf[0, :t].mean(axis=0), rtol=0, atol=1e-6)
    assert np.allclose(out[1], vf[1, :20].mean(axis=0), rtol=0, atol=1e-6)


def test_attention_against_scipy_softmax():
    s, h, d, t = 2, 4, 32, 130
    q = np.random.default_rng(5).standard_normal((s, h, d)).astype(np.float32) * 3
    k = synth.kv_f16((s, t, h, d), seed=6)
    v = synth.kv_f16((s, t, h, d), seed=7)
    n_ctx = [130, 77]
    scale = 1.0 / np.sqrt(d)
    got_c = oracle_c.attn_decode(q, k, v, n_ctx, scale)
    got_np = oracle_np.attn_decode(q, k, v, n_ctx, scale)
    kf = k.view(np.float16).astype(np.float64)
    vf = v.view(np.float16).astype(np.float64)
    for si in range(s):
        n = n_ctx[si]
        for hi in range(h):
            p = scipy.special.softmax(kf[si, :n, hi] @ q[si, hi].astype(np.float64) * scale)
            want = p @ vf[si, :n, hi]
            assert np.allclose(got_c[si, hi], want, rtol=1e-6, atol=1e-7)
            assert np.allclose(got_np[si, hi], want, rtol=1e-6, atol=1e-7)


def test_attention_large_scores_do_not_overflow():
    q = np.full((1, 1, 8), 60.0, dtype=np.float32)
    k = (np.ones((1, 4, 1, 8), dtype=np.float16) * np.array([1, 2, 3, 4], dtype=np.float16)[None, :, None, None]).view(np.uint16)
    v = synth.kv_f16((1, 4, 1, 8), seed=3)
    out = oracle_c.attn_decode(q, k, v, [4], 1.0)
    assert np.all(np.isfinite(out))
    # score gaps of 480: the last token takes all the weight
    assert np.allclose(out[0, 0], v[0, 3, 0].view(np.float16).astype(np.float32), atol=1e-6)


def test_flat_kv_shadow():
    kv = oracle_np.FlatKV(2, 2, 4, 5)
    rows = synth.kv_f16((3, 2, 4), seed=1)
    kv.append(rows, rows + 1, [0, 1, 0])
    assert kv.len.tolist() == [2, 1]
    k, v = kv.gather(0, 0, 2)
    assert np.array_equal(k, rows[[0, 2]]) and np.array_equal(v, rows[[0, 2]] + 1)


def test_rmsnorm_rope_swiglu_closed_forms():
    x = np.array([3.0, -4.0, 0.0, 0.0], dtype=np.float32)
    w = np.array([1.0, 2.0, 3.0, 4.0], dtype=np.float32)
    # mean square = 25/4, eps 0 -> x / 2.5
    assert np.allclose(oracle_c.rmsnorm(x, w, 0.0), [1.2, -3.2, 0, 0], atol=1e-7)
    assert np.allclose(oracle_np.rmsnorm(x, w, 0.0), [1.2, -3.2, 0, 0], atol=1e-7)
    # rope: position 0 is the identity; a rotation preserves pair norms; pair i turns by pos * base^(-2i/dim)
    v = np.random.default_rng(2).standard_normal((2, 8)).astype(np.float32)
    assert np.array_equal(oracle_c.rope(v, 0), v)
    r = oracle_c.rope(v, 7, 10000.0)
    assert np.allclose(r, oracle_np.rope(v, 7, 10000.0), atol=1e-6)
    assert np.allclose(r[:, 0::2] ** 2 + r[:, 1::2] ** 2, v[:, 0::2] ** 2 + v[:, 1::2] ** 2, atol=1e-5)
    ang = np.arctan2(r[0, 3], r[0, 2]) - np.arctan2(v[0, 3], v[0, 2])
    assert np.isclose(np.mod(ang, 2 * np.pi), np.mod(7 * 10000.0 ** (-2.0 / 8), 2 * np.pi), atol=1e-5)
    # swiglu at known points: silu(0)=0, silu(x) -> x for large x
    g = np.array([0.0, 30.0, -30.0, 1.0], dtype=np.float32)
    u = np.array([5.0, 2.0, 2.0, 1.0], dtype=np.float32)
    want = [0.0, 60.0, 0.0, 1.0 / (1.0 + np.exp(-1.0))]
    assert np.allclose(oracle_c.swiglu(g, u), want, atol=1e-5)
    assert np.allclose(oracle_np.swiglu(g, u), want, atol=1e-5)
    assert oracle_c.argmax(np.array([1.0, 7.0, 7.0, 3.0])) == 1
