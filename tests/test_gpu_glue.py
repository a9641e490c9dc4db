"""GPU parity of the decoder glue ops (fp32) against the CPU oracle; tolerance 1e-5 relative unless noted."""
import numpy as np
import pytest

from oracle import oracle_c, oracle_np
from skainet_amd import runtime, synth

pytestmark = pytest.mark.gpu


def test_rmsnorm(hip):
    rows, n = 5, 4096
    x = np.random.default_rng(0).standard_normal((rows, n)).astype(np.float32) * 3
    w = np.random.default_rng(1).standard_normal(n).astype(np.float32)
    y = hip.alloc(x.nbytes)
    hip.rmsnorm(hip.to_device(x), hip.to_device(w), rows, n, 1e-5, y)
    got = y.download(np.float32, x.size).reshape(x.shape)
    want = np.stack([oracle_c.rmsnorm(x[r], w, 1e-5) for r in range(rows)])
    assert oracle_np.rel_err(got, want) <= 1e-5


def test_rope(hip):
    rows, n_head, dim = 3, 4, 128
    x = np.random.default_rng(2).standard_normal((rows, n_head, dim)).astype(np.float32)
    xd = hip.to_device(x)
    hip.rope(xd, rows, n_head, dim, 637, 10000.0)
    got = xd.download(np.float32, x.size).reshape(x.shape)
    want = np.stack([oracle_c.rope(x[r], 637 + r, 10000.0) for r in range(rows)])
    # the angle is formed and reduced in double: what is left is the fp32 rounding of the rotation itself
    assert np.max(np.abs(got - want)) <= 2e-6
    # far into a long context the angle of the first pairs is thousands of radians: still the fp32 rotation's rounding
    xd = hip.to_device(x)
    hip.rope(xd, rows, n_head, dim, 8189, 10000.0)
    want = np.stack([oracle_c.rope(x[r], 8189 + r, 10000.0) for r in range(rows)])
    assert np.max(np.abs(xd.download(np.float32, x.size).reshape(x.shape) - want)) <= 2e-6
    xd = hip.to_device(x)
    hip.rope(xd, rows, n_head, dim, 0, 10000.0)
    assert np.array_equal(xd.download(np.float32, x.size).reshape(x.shape)[0], x[0])  # position 0: identity


def test_swiglu_add_argmax(hip):
    n = 11008
    g = np.random.default_rng(3).standard_normal(n).astype(np.float32) * 4
    u = np.random.default_rng(4).standard_normal(n).astype(np.float32)
    o = hip.alloc(4 * n)
    hip.swiglu(hip.to_device(g), hip.to_device(u), n, o)
    assert oracle_np.rel_err(o.download(np.float32, n), oracle_c.swiglu(g, u)) <= 1e-5
    yd = hip.to_device(g)
    hip.add_inplace(yd, hip.to_device(u), n)
    assert np.array_equal(yd.download(np.float32, n), g + u)
    idx = hip.alloc(16)
    x = np.random.default_rng(5).standard_normal(32000).astype(np.float32)
    x[[17, 20001]] = x.max() + 1.0  # tie: the first maximum wins
    hip.argmax(hip.to_device(x), x.size, idx)
    assert int(idx.download(np.int32, 1)[0]) == oracle_c.argmax(x) == 17


def test_float_conversions(hip):
    x = np.concatenate([
        np.random.default_rng(6).standard_normal(100000).astype(np.float32) * 100,
        np.array([0.0, -0.0, 65504.0, 65520.0, 1e-8, 6e-8, 2.0 ** -25, 1e30], dtype=np.float32),
    ])
    out = hip.alloc(2 * x.size)
    hip.f32_to_f16(hip.to_device(x), x.size, out)
    assert np.array_equal(out.download(np.uint16, x.size), oracle_c.f2h(x))
    hip.f32_to_bf16(hip.to_device(x), x.size, out)
    assert np.array_equal(out.download(np.uint16, x.size), synth.f32_to_bf16_bits(x))
