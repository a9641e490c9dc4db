"""GPU: skn_attn_decode_static -- decode attention with the split scratch in a fixed device array of the library --
against skn_attn_decode on the same cache: two calls in a row, the second on a smaller cache and shorter contexts,
so that what the first call left in the shared array is what the second one starts from.  Bar: 1e-3 of
max(|ref|, 1e-3 max|ref|), the attention tolerance; the oracle is checked on the small case as well."""
import numpy as np
import pytest

from oracle import oracle_c, oracle_np
from skainet_amd import runtime, synth

pytestmark = pytest.mark.gpu


def _filled_cache(hip, n_seq, n_head, dim, page, lens, seed):
    kv = hip.kv_cache(n_seq, n_head, dim, page, max(lens) + page)
    ks, vs = [], []
    for s, n in enumerate(lens):
        k = synth.kv_f16((n, n_head, dim), seed=seed + 2 * s)
        v = synth.kv_f16((n, n_head, dim), seed=seed + 2 * s + 1)
        kv.append_run(s, hip.to_device(k), hip.to_device(v), n)
        ks.append(k)
        vs.append(v)
    return kv, ks, vs


def _both(hip, kv, n_seq, n_head, dim, seed):
    q = np.random.default_rng(seed).standard_normal((n_seq, n_head, dim)).astype(np.float32)
    qd = hip.to_device(q)
    out_ref, out_new = hip.alloc(q.nbytes), hip.alloc(q.nbytes)
    hip.memset(out_new, 0xFF, q.nbytes)
    kv.attn_decode(qd, out_ref, dim ** -0.5)
    kv.attn_decode_static(qd, out_new, dim ** -0.5)
    ref = out_ref.download(np.float32, q.size).reshape(q.shape)
    new = out_new.download(np.float32, q.size).reshape(q.shape)
    return q, ref, new


def test_static_scratch_attention_matches_the_allocating_entry_point(hip):
    # first call: many splits per (sequence, head) pair
    lens = [3000, 2500, 1777, 4096]
    kv, _, _ = _filled_cache(hip, 4, 8, 128, 256, lens, seed=100)
    q, ref, new = _both(hip, kv, 4, 8, 128, seed=7)
    assert np.all(np.isfinite(new))
    assert oracle_np.rel_err(new, ref) <= 1e-3
    kv.free()
    # second call: smaller cache, fewer pairs, fewer splits, another head_dim
    lens2 = [300, 129]
    kv2, ks, vs = _filled_cache(hip, 2, 4, 64, 16, lens2, seed=200)
    q2, ref2, new2 = _both(hip, kv2, 2, 4, 64, seed=8)
    assert oracle_np.rel_err(new2, ref2) <= 1e-3
    pad = max(lens2)
    kk = np.zeros((2, pad, 4, 64), np.uint16)
    vv = np.zeros_like(kk)
    for s, n in enumerate(lens2):
        kk[s, :n], vv[s, :n] = ks[s], vs[s]
    want = oracle_c.attn_decode(q2, kk, vv, lens2, 64 ** -0.5)
    assert oracle_np.rel_err(new2, want) <= 1e-3
    # and a third, again larger than the second, on the same array
    q3, ref3, new3 = _both(hip, kv2, 2, 4, 64, seed=9)
    assert oracle_np.rel_err(new3, ref3) <= 1e-3
    kv2.free()


def test_static_scratch_attention_rejects_what_does_not_fit(hip):
    kv = hip.kv_cache(64, 128, 64, 16, 16)  # 8192 pairs: beyond the 4096 counters
    buf = hip.alloc(64 * 128 * 64 * 4)
    with pytest.raises(runtime.SknError) as e:
        kv.attn_decode_static(buf, buf, 1.0)
    assert e.value.code == runtime.ERR_SHAPE and "4096" in e.value.message
    kv.free()
