"""GPU parity: paged KV cache append / gather (bit-exact vs a flat shadow) and decode attention (<= 1e-3)."""
import numpy as np
import pytest

from oracle import oracle_c, oracle_np
from skainet_amd import runtime, synth

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _gather(hip, kv, seq, t0, t1):
    n = (t1 - t0) * kv.n_head * kv.head_dim
    kd, vd = hip.alloc(max(2 * n, 16)), hip.alloc(max(2 * n, 16))
    kv.gather(seq, t0, t1, kd, vd)
    shape = (t1 - t0, kv.n_head, kv.head_dim)
    return kd.download(np.uint16, n).reshape(shape), vd.download(np.uint16, n).reshape(shape)


def test_append_gather_round_trip_across_pages(hip):
    n_seq, n_head, dim, page, cap = 3, 4, 64, 16, 80
    kv = hip.kv_cache(n_seq, n_head, dim, page, cap)
    shadow = oracle_np.FlatKV(n_seq, n_head, dim, cap)
    rng = np.random.default_rng(0)
    step = 0
    # ragged growth: sequences advance at different rates and cross page boundaries at different steps
    while shadow.len.max() < 50:
        ids = [s for s in range(n_seq) if rng.random() < (0.9, 0.5, 0.3)[s]]
        if step % 7 == 3:
            ids = ids + [0, 0]  # the same sequence listed several times in one call
        if not ids:
            continue
        k = synth.kv_f16((len(ids), n_head, dim), seed=1000 + step)
        v = synth.kv_f16((len(ids), n_head, dim), seed=2000 + step)
        kv.append(hip.to_device(k), hip.to_device(v), ids)
        shadow.append(k, v, ids)
        step += 1
    for s in range(n_seq):
        n = int(shadow.len[s])
        assert kv.length(s) == n
        gk, gv = _gather(hip, kv, s, 0, n)
        wk, wv = shadow.gather(s, 0, n)
        assert np.array_equal(gk, wk) and np.array_equal(gv, wv)
        if n > 20:
            gk, gv = _gather(hip, kv, s, 15, 18)  # a range straddling the first page boundary
            wk, wv = shadow.gather(s, 15, 18)
            assert np.array_equal(gk, wk) and np.array_equal(gv, wv)
    kv.free()


def test_append_run_page_boundaries_and_capacity(hip):
    n_head, dim, page, cap = 2, 128, 256, 8192
    kv = hip.kv_cache(1, n_head, dim, page, cap)
    k = synth.kv_f16((cap, n_head, dim), seed=3)
    v = synth.kv_f16((cap, n_head, dim), seed=4)
    kd, vd = hip.to_device(k), hip.to_device(v)
    row = n_head * dim * 2
    kv.append_run(0, kd, vd, 255)
    kv.append(kd.ptr + 255 * row, vd.ptr + 255 * row, [0])  # t = 255 -> last slot of page 0
    kv.append(kd.ptr + 256 * row, vd.ptr + 256 * row, [0])  # t = 256 -> first slot of a new page
    kv.append_run(0, kd.ptr + 257 * row, vd.ptr + 257 * row, cap - 257 - 1)
    kv.append(kd.ptr + (cap - 1) * row, vd.ptr + (cap - 1) * row, [0])  # t = 8191: the last token that fits
    assert kv.length(0) == cap
    gk, gv = _gather(hip, kv, 0, 0, cap)
    assert np.array_equal(gk, k) and np.array_equal(gv, v)
    with pytest.raises(runtime.SknError) as e:
        kv.append(kd, vd, [0])
    assert e.value.code == runtime.ERR_POOL
    with pytest.raises(runtime.SknError) as e:
        kv.append_run(0, kd, vd, 1)
    assert e.value.code == runtime.ERR_POOL
    assert kv.length(0) == cap
    # reset returns the pages; the sequence can grow again and holds the new data
    kv.reset(0)
    assert kv.length(0) == 0
    kv.append_run(0, vd, kd, 300)
    gk, gv = _gather(hip, kv, 0, 0, 300)
    assert np.array_equal(gk, v[:300]) and np.array_equal(gv, k[:300])
    kv.free()


def test_kv_argument_errors(hip):
    kv = hip.kv_cache(2, 2, 64, 16, 32)
    buf = hip.alloc(4096)
    with pytest.raises(runtime.SknError) as e:
        kv.append(buf, buf, [2])
    assert e.value.code == runtime.ERR_RANGE
    with pytest.raises(runtime.SknError) as e:
        kv.gather(0, 0, 1, buf, buf)  # nothing cached yet
    assert e.value.code == runtime.ERR_RANGE
    with pytest.raises(runtime.SknError) as e:
        kv.length(5)
    assert e.value.code == runtime.ERR_RANGE
    with pytest.raises(runtime.SknError) as e:
        hip.kv_cache(1, 1, 12, 16, 32)  # head_dim not a multiple of 8
    assert e.value.code == runtime.ERR_SHAPE
    kv.append(buf, buf, [])  # empty append is a no-op
    kv.free()


def _fill(hip, kv, lens, seed):
    n_seq, n_head, dim = kv.n_seq, kv.n_head, kv.head_dim
    cap = max(lens)
    k = synth.kv_f16((n_seq, cap, n_head, dim), seed=seed)
    v = synth.kv_f16((n_seq, cap, n_head, dim), seed=seed + 1)
    for s in range(n_seq):
        if lens[s]:
            kv.append_run(s, hip.to_device(k[s, : lens[s]]), hip.to_device(v[s, : lens[s]]), lens[s])
    return k, v


@pytest.mark.parametrize(
    "n_seq,n_head,dim,page,lens",
    [
        (2, 4, 128, 256, [300, 77]),
        (3, 2, 64, 16, [1, 64, 65]),
        (1, 32, 128, 256, [640]),
        (2, 2, 256, 32, [100, 33]),
        (4, 8, 128, 256, [1024, 0, 513, 255]),
    ],
)
def test_attention_vs_oracle(hip, n_seq, n_head, dim, page, lens):
    kv = hip.kv_cache(n_seq, n_head, dim, page, max(max(lens), page))
    k, v = _fill(hip, kv, lens, seed=11)
    q = np.random.default_rng(5).standard_normal((n_seq, n_head, dim)).astype(np.float32)
    scale = 1.0 / np.sqrt(dim)
    out = hip.alloc(q.nbytes)
    kv.attn_decode(hip.to_device(q), out, scale)
    got = out.download(np.float32, q.size).reshape(q.shape)
    want = oracle_c.attn_decode(q, k, v, lens, scale)
    for s in range(n_seq):
        if lens[s] == 0:
            assert np.all(got[s] == 0.0)
        else:
            assert oracle_np.rel_err(got[s], want[s]) <= TOL
    # explicit shorter contexts
    short = [max(0, n // 2) for n in lens]
    kv.attn_decode(hip.to_device(q), out, scale, n_ctx=short)
    got = out.download(np.float32, q.size).reshape(q.shape)
    want = oracle_c.attn_decode(q, k, v, short, scale)
    for s in range(n_seq):
        if short[s]:
            assert oracle_np.rel_err(got[s], want[s]) <= TOL
    with pytest.raises(runtime.SknError) as e:
        kv.attn_decode(hip.to_device(q), out, scale, n_ctx=[n + 1 for n in lens])
    assert e.value.code == runtime.ERR_RANGE
    kv.free()


def test_attention_closed_forms(hip):
    n_seq, n_head, dim, t = 2, 4, 128, 200
    kv = hip.kv_cache(n_seq, n_head, dim, 64, 256)
    k = synth.kv_f16((n_seq, t, n_head, dim), seed=1)
    v = synth.kv_f16((n_seq, t, n_head, dim), seed=2)
    ku = np.broadcast_to(k[:, :1], k.shape).copy()  # identical keys -> uniform weights -> mean of V
    for s in range(n_seq):
        kv.append_run(s, hip.to_device(ku[s]), hip.to_device(v[s]), t)
    q = np.random.default_rng(3).standard_normal((n_seq, n_head, dim)).astype(np.float32)
    out = hip.alloc(q.nbytes)
    kv.attn_decode(hip.to_device(q), out, 0.1)
    got = out.download(np.float32, q.size).reshape(q.shape)
    mean_v = v.view(np.float16).astype(np.float64).mean(axis=1)
    assert np.allclose(got, mean_v, rtol=0, atol=2e-6 + 1e-3 * np.abs(mean_v).max() * 1e-3)
    # one token -> its V row; large score gaps must not overflow
    kv.attn_decode(hip.to_device(q * 50.0), out, 1.0, n_ctx=[1, 1])
    got = out.download(np.float32, q.size).reshape(q.shape)
    assert np.array_equal(got, v[:, 0].view(np.float16).astype(np.float32))
    kv.free()


def test_benchmark_shape_step(hip):
    """8 sequences x 32 heads x 128, 256-token pages: 4095 cached tokens, append one, attend over 4096."""
    n_seq, n_head, dim = 8, 32, 128
    kv = hip.kv_cache(n_seq, n_head, dim, 256, 8192)
    k, v = _fill(hip, kv, [4095] * n_seq, seed=21)
    k1 = synth.kv_f16((n_seq, n_head, dim), seed=31)
    v1 = synth.kv_f16((n_seq, n_head, dim), seed=32)
    kv.append(hip.to_device(k1), hip.to_device(v1), list(range(n_seq)))
    q = np.random.default_rng(9).standard_normal((n_seq, n_head, dim)).astype(np.float32)
    out = hip.alloc(q.nbytes)
    kv.attn_decode(hip.to_device(q), out, 1.0 / np.sqrt(dim))
    got = out.download(np.float32, q.size).reshape(q.shape)
    kf = np.concatenate([k, k1[:, None]], axis=1)
    vf = np.concatenate([v, v1[:, None]], axis=1)
    want = oracle_c.attn_decode(q, kf, vf, [4096] * n_seq, 1.0 / np.sqrt(dim))
    assert oracle_np.rel_err(got, want) <= TOL
    # the appended token is stored bit-exactly at position 4095
    gk, gv = _gather(hip, kv, 5, 4095, 4096)
    assert np.array_equal(gk[0], k1[5]) and np.array_equal(gv[0], v1[5])
    kv.free()


def test_attention_split_counts_and_repeated_launches(hip):
    """Every split count gives the same answer, launch after launch: the per-(sequence, head) counters that
    elect the merging workgroup are left at zero by each launch.  Pages of 48 tokens (not a power of two)."""
    n_seq, n_head, dim = 3, 4, 128
    lens = [700, 5, 193]
    kv = hip.kv_cache(n_seq, n_head, dim, 48, 720)
    k, v = _fill(hip, kv, lens, seed=41)
    q = np.random.default_rng(6).standard_normal((n_seq, n_head, dim)).astype(np.float32)
    scale = 1.0 / np.sqrt(dim)
    want = oracle_c.attn_decode(q, k, v, lens, scale)
    out = hip.alloc(q.nbytes)
    qd = hip.to_device(q)
    try:
        for splits in (1, 2, 3, 7, 11, 64, 0, 5, 5, 5):
            hip.set_option("attn.splits", splits)
            out.upload(np.full(q.shape, np.nan, np.float32))
            kv.attn_decode(qd, out, scale)
            got = out.download(np.float32, q.size).reshape(q.shape)
            assert oracle_np.rel_err(got, want) <= TOL, splits
    finally:
        hip.set_option("attn.splits", 0)
    kv.free()


@pytest.mark.parametrize(
    "n_head,dim,page,cached,n_queries",
    [
        (4, 128, 256, 300, 300),   # a whole prompt: row t sees t + 1 tokens
        (2, 64, 16, 70, 70),
        (3, 128, 48, 130, 45),     # the last 45 tokens of 130 (pages of 48: tiles straddle pages)
        (2, 128, 32, 33, 1),       # a single row = decode attention
        (8, 64, 64, 257, 200),
    ],
)
def test_prefill_attention_vs_oracle(hip, n_head, dim, page, cached, n_queries):
    """skn_attn_prefill: causal attention of the last n_queries tokens of a sequence, against the oracle run
    once per row with that row's context length."""
    kv = hip.kv_cache(2, n_head, dim, page, max(cached, page) + page)
    k, v = _fill(hip, kv, [5, cached], seed=51)   # sequence 1 is the one attended to; 0 holds something else
    q = np.random.default_rng(8).standard_normal((n_queries, n_head, dim)).astype(np.float32) * 2.0
    scale = 1.0 / np.sqrt(dim)
    out = hip.alloc(q.nbytes)
    out.upload(np.full(q.shape, np.nan, np.float32))
    kv.attn_prefill(1, hip.to_device(q), n_queries, out, scale)
    got = out.download(np.float32, q.size).reshape(q.shape)
    ctx_len = [cached - n_queries + t + 1 for t in range(n_queries)]
    kk = np.broadcast_to(k[1][None], (n_queries,) + k[1].shape)
    vv = np.broadcast_to(v[1][None], (n_queries,) + v[1].shape)
    want = oracle_c.attn_decode(q, np.ascontiguousarray(kk), np.ascontiguousarray(vv), ctx_len, scale)
    for t in range(n_queries):
        assert oracle_np.rel_err(got[t], want[t]) <= TOL, t
    # the same rows through the decode kernel (sequence 1, explicit context of the last row)
    if n_queries == 1:
        out2 = hip.alloc(2 * n_head * dim * 4)
        q2 = np.zeros((2, n_head, dim), np.float32)
        q2[1] = q[0]
        kv.attn_decode(hip.to_device(q2), out2, scale, n_ctx=[0, cached])
        dec = out2.download(np.float32, 2 * n_head * dim).reshape(2, n_head, dim)[1]
        assert oracle_np.rel_err(got[0], dec) <= TOL
    kv.free()


def test_prefill_attention_arguments_and_closed_form(hip):
    n_head, dim, tok = 2, 128, 96
    kv = hip.kv_cache(1, n_head, dim, 32, 128)
    k = synth.kv_f16((1, tok, n_head, dim), seed=61)
    v = synth.kv_f16((1, tok, n_head, dim), seed=62)
    ku = np.broadcast_to(k[:, :1], k.shape).copy()  # identical keys: row t returns the mean of V[0 : t + 1]
    kv.append_run(0, hip.to_device(ku[0]), hip.to_device(v[0]), tok)
    q = np.random.default_rng(9).standard_normal((tok, n_head, dim)).astype(np.float32)
    out = hip.alloc(q.nbytes)
    kv.attn_prefill(0, hip.to_device(q), tok, out, 0.3)
    got = out.download(np.float32, q.size).reshape(q.shape)
    vf = v[0].view(np.float16).astype(np.float64)
    means = np.cumsum(vf, axis=0) / np.arange(1, tok + 1)[:, None, None]
    assert np.abs(got - means).max() <= 1e-3 * np.abs(means).max() * 1e-3 + 2e-6
    with pytest.raises(runtime.SknError) as e:
        kv.attn_prefill(0, hip.to_device(q), tok + 1, out, 0.3)  # more rows than cached tokens
    assert e.value.code == runtime.ERR_RANGE
    with pytest.raises(runtime.SknError) as e:
        kv.attn_prefill(3, hip.to_device(q), 1, out, 0.3)
    assert e.value.code == runtime.ERR_RANGE
    kv.attn_prefill(0, hip.to_device(q), 0, out, 0.3)  # no rows: a no-op
    kv256 = hip.kv_cache(1, 1, 256, 32, 64)
    kv256.append_run(0, hip.alloc(256 * 2 * 4), hip.alloc(256 * 2 * 4), 4)
    with pytest.raises(runtime.SknError) as e:
        kv256.attn_prefill(0, hip.to_device(q), 2, out, 0.3)
    assert e.value.code == runtime.ERR_SHAPE
    kv256.free()
    kv.free()
