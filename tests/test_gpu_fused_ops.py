"""GPU: every fused form of the decoder's matvec as an operation of its own against the CPU oracle, at the bound of an
operation: 1e-3 of max(|ref|, 1e-3 max|ref|), stated here before any measurement.  One launch each through the C ABI's
test hook: [RMSNorm + q,k,v + rotary + cache store], [+= W . x], [RMSNorm + gate,up + SwiGLU], plain stores; every
weight format that has a fused kernel; the 7B shapes for Q4_K."""
import numpy as np
import pytest

from oracle import oracle_c, oracle_np
from skainet_amd import synth

pytestmark = pytest.mark.gpu
TOL = 1e-3
FUSED_TYPES = [synth.Q4_K, synth.Q5_K, synth.Q4_0, synth.Q4_1, synth.Q5_0, synth.Q5_1, synth.IQ4_NL, synth.Q6_K, synth.Q8_0,
               synth.IQ4_XS, synth.Q2_K, synth.Q3_K, synth.Q8_K, synth.TQ2_0, synth.TQ1_0]
STORE, ADD, SWIGLU, ROPE = 0, 1, 2, 3


def _norm(x, g, eps):
    return oracle_c.rmsnorm(x, g, eps)


@pytest.mark.parametrize("qtype", FUSED_TYPES)
def test_norm_qkv_rope_cache_store(hip, qtype):
    heads, dim, k, page = 4, 128, 1024, 16
    h = heads * dim
    pos = 21  # second page of the cache
    wq, wk, wv = (synth.weight(qtype, h, k, seed=40 + i) for i in range(3))
    x = synth.activation_f32(k, seed=50) * 3.0
    g = (1.0 + 0.1 * np.random.default_rng(51).standard_normal(k)).astype(np.float32)
    kv = hip.kv_cache(1, heads, dim, page, 64)
    kv.append_run(0, hip.to_device(synth.kv_f16((pos, heads, dim), seed=52)), hip.to_device(synth.kv_f16((pos, heads, dim), seed=53)), pos)
    y = hip.alloc(4 * h)
    pos_dev = hip.alloc(16)
    hip.test_fused_matvec(qtype, ROPE, [(hip.to_device(wq), h), (hip.to_device(wk), h), (hip.to_device(wv), h)], k,
                          hip.to_device(x), hip.to_device(g), 1e-5, y, kv=kv, pos_dev=pos_dev)
    xn = _norm(x, g, 1e-5)
    q = oracle_c.rope(oracle_c.matvec_q(qtype, wq, h, k, xn).reshape(heads, dim), pos, 10000.0)
    kk = oracle_c.rope(oracle_c.matvec_q(qtype, wk, h, k, xn).reshape(heads, dim), pos, 10000.0)
    vv = oracle_c.matvec_q(qtype, wv, h, k, xn).reshape(heads, dim)
    assert oracle_np.rel_err(y.download(np.float32, h).reshape(heads, dim), q) <= TOL
    assert kv.length(0) == pos + 1
    ko, vo = hip.alloc(2 * h), hip.alloc(2 * h)
    kv.gather(0, pos, pos + 1, ko, vo)
    got_k = ko.download(np.uint16, h).view(np.float16).astype(np.float32).reshape(heads, dim)
    got_v = vo.download(np.uint16, h).view(np.float16).astype(np.float32).reshape(heads, dim)
    # the cache holds fp16: half an fp16 unit in the last place (2^-11 relative) on top of the operation's own error
    assert oracle_np.rel_err(got_k, kk) <= TOL
    assert oracle_np.rel_err(got_v, vv) <= TOL
    kv.free()


@pytest.mark.parametrize("qtype", FUSED_TYPES)
def test_norm_gate_up_swiglu(hip, qtype):
    f, k = 384, 1024
    wg, wu = synth.weight(qtype, f, k, seed=60), synth.weight(qtype, f, k, seed=61)
    x = synth.activation_f32(k, seed=62)
    g = (1.0 + 0.1 * np.random.default_rng(63).standard_normal(k)).astype(np.float32)
    y = hip.alloc(4 * f)
    hip.test_fused_matvec(qtype, SWIGLU, [(hip.to_device(wg), f), (hip.to_device(wu), f)], k, hip.to_device(x), hip.to_device(g),
                          1e-5, y)
    xn = _norm(x, g, 1e-5)
    want = oracle_c.swiglu(oracle_c.matvec_q(qtype, wg, f, k, xn), oracle_c.matvec_q(qtype, wu, f, k, xn))
    assert oracle_np.rel_err(y.download(np.float32, f), want) <= TOL


@pytest.mark.parametrize("qtype", FUSED_TYPES)
def test_residual_add_and_plain_store(hip, qtype):
    n, k = 256, 2048
    w = synth.weight(qtype, n, k, seed=70)
    x = synth.activation_f32(k, seed=71)
    res = synth.activation_f32(n, seed=72) * 50.0
    want = oracle_c.matvec_q(qtype, w, n, k, x).astype(np.float64)
    wd, xd = hip.to_device(w), hip.to_device(x)
    y = hip.to_device(res)
    hip.test_fused_matvec(qtype, ADD, [(wd, n)], k, xd, None, 0.0, y)
    assert oracle_np.rel_err(y.download(np.float32, n), want + res) <= TOL
    # what was added is the product itself to the bound (the residual must not hide its error)
    assert oracle_np.rel_err(y.download(np.float32, n).astype(np.float64) - res, want) <= 2 * TOL
    y2 = hip.alloc(4 * n)
    hip.test_fused_matvec(qtype, STORE, [(wd, n)], k, xd, None, 0.0, y2)
    assert oracle_np.rel_err(y2.download(np.float32, n), want) <= TOL


def test_q4k_fused_forms_at_the_7b_shapes(hip):
    """hidden 4096, FFN 11008, 32 heads x 128: the four launches of a Q4_K layer, sampled rows of the oracle."""
    hdim, ffn, heads, dim = 4096, 11008, 32, 128
    rng = np.random.default_rng(80)
    x = synth.activation_f32(hdim, seed=81)
    g = (1.0 + 0.1 * rng.standard_normal(hdim)).astype(np.float32)
    xn = _norm(x, g, 1e-5)
    # gate / up + SwiGLU
    wg, wu = synth.weight(synth.Q4_K, ffn, hdim, seed=82), synth.weight(synth.Q4_K, ffn, hdim, seed=83)
    y = hip.alloc(4 * ffn)
    hip.test_fused_matvec(synth.Q4_K, SWIGLU, [(hip.to_device(wg), ffn), (hip.to_device(wu), ffn)], hdim, hip.to_device(x),
                          hip.to_device(g), 1e-5, y)
    want = oracle_c.swiglu(oracle_c.matvec_q(synth.Q4_K, wg, ffn, hdim, xn), oracle_c.matvec_q(synth.Q4_K, wu, ffn, hdim, xn))
    mid = y.download(np.float32, ffn)
    assert oracle_np.rel_err(mid, want) <= TOL
    # down + residual (k = 11008: three steps, the last one partly filled)
    wd = synth.weight(synth.Q4_K, hdim, ffn, seed=84)
    res = synth.activation_f32(hdim, seed=85)
    yr = hip.to_device(res)
    hip.test_fused_matvec(synth.Q4_K, ADD, [(hip.to_device(wd), hdim)], ffn, hip.to_device(want.astype(np.float32)), None, 0.0, yr)
    want_d = oracle_c.matvec_q(synth.Q4_K, wd, hdim, ffn, want.astype(np.float32)).astype(np.float64) + res
    assert oracle_np.rel_err(yr.download(np.float32, hdim), want_d) <= TOL
    # q, k, v + rotary + cache store at a position on a page boundary
    wq, wk, wv = (synth.weight(synth.Q4_K, hdim, hdim, seed=86 + i) for i in range(3))
    pos = 256
    kv = hip.kv_cache(1, heads, dim, 256, 512)
    kv.append_run(0, hip.to_device(synth.kv_f16((pos, heads, dim), seed=90)), hip.to_device(synth.kv_f16((pos, heads, dim), seed=91)), pos)
    yq = hip.alloc(4 * hdim)
    hip.test_fused_matvec(synth.Q4_K, ROPE, [(hip.to_device(wq), hdim), (hip.to_device(wk), hdim), (hip.to_device(wv), hdim)], hdim,
                          hip.to_device(x), hip.to_device(g), 1e-5, yq, kv=kv, pos_dev=hip.alloc(16))
    q = oracle_c.rope(oracle_c.matvec_q(synth.Q4_K, wq, hdim, hdim, xn).reshape(heads, dim), pos, 10000.0)
    assert oracle_np.rel_err(yq.download(np.float32, hdim).reshape(heads, dim), q) <= TOL
    ko, vo = hip.alloc(2 * hdim), hip.alloc(2 * hdim)
    kv.gather(0, pos, pos + 1, ko, vo)
    kk = oracle_c.rope(oracle_c.matvec_q(synth.Q4_K, wk, hdim, hdim, xn).reshape(heads, dim), pos, 10000.0)
    vv = oracle_c.matvec_q(synth.Q4_K, wv, hdim, hdim, xn).reshape(heads, dim)
    assert oracle_np.rel_err(ko.download(np.uint16, hdim).view(np.float16).astype(np.float32).reshape(heads, dim), kk) <= TOL
    assert oracle_np.rel_err(vo.download(np.uint16, hdim).view(np.float16).astype(np.float32).reshape(heads, dim), vv) <= TOL
    kv.free()


@pytest.mark.parametrize("pos", [21, 256, 8189])
@pytest.mark.parametrize("table", [0, 1])
@pytest.mark.parametrize("kv_heads", [4, 2])
def test_rotary_epilogue_with_and_without_the_frequency_table(hip, pos, table, kv_heads):
    """The rotary epilogue takes a pair's frequency either from a device table of doubles (what every decoder launch
    passes: base^(-2i/d) formed on the host) or from exp2 inside the kernel.  Both branches, at a position on the
    second page, on a page boundary and near 8192, with as many K / V heads as query heads and with fewer (the k
    and v segments then have fewer rows than q, which moves the table index), against the oracle's rotation."""
    heads, dim, k, page = 4, 128, 1024, 256
    hq, hkv = heads * dim, kv_heads * dim
    wq = synth.weight(synth.Q4_K, hq, k, seed=140)
    wk, wv = synth.weight(synth.Q4_K, hkv, k, seed=141), synth.weight(synth.Q4_K, hkv, k, seed=142)
    x = synth.activation_f32(k, seed=150) * 3.0
    g = (1.0 + 0.1 * np.random.default_rng(151).standard_normal(k)).astype(np.float32)
    kv = hip.kv_cache(1, kv_heads, dim, page, 8192)
    fill_k = hip.to_device(synth.kv_f16((pos, kv_heads, dim), seed=152))
    kv.append_run(0, fill_k, fill_k, pos)
    y = hip.alloc(4 * hq)
    hip.set_option("test.rope_table", table)
    try:
        hip.test_fused_matvec(synth.Q4_K, ROPE, [(hip.to_device(wq), hq), (hip.to_device(wk), hkv), (hip.to_device(wv), hkv)], k,
                              hip.to_device(x), hip.to_device(g), 1e-5, y, kv=kv, pos_dev=hip.alloc(16))
    finally:
        hip.set_option("test.rope_table", 0)
    xn = _norm(x, g, 1e-5)
    q = oracle_c.rope(oracle_c.matvec_q(synth.Q4_K, wq, hq, k, xn).reshape(heads, dim), pos, 10000.0)
    kk = oracle_c.rope(oracle_c.matvec_q(synth.Q4_K, wk, hkv, k, xn).reshape(kv_heads, dim), pos, 10000.0)
    vv = oracle_c.matvec_q(synth.Q4_K, wv, hkv, k, xn).reshape(kv_heads, dim)
    assert oracle_np.rel_err(y.download(np.float32, hq).reshape(heads, dim), q) <= TOL
    ko, vo = hip.alloc(2 * hkv), hip.alloc(2 * hkv)
    kv.gather(0, pos, pos + 1, ko, vo)
    assert oracle_np.rel_err(ko.download(np.uint16, hkv).view(np.float16).astype(np.float32).reshape(kv_heads, dim), kk) <= TOL
    assert oracle_np.rel_err(vo.download(np.uint16, hkv).view(np.float16).astype(np.float32).reshape(kv_heads, dim), vv) <= TOL
    kv.free()
