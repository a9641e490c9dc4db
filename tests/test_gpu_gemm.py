"""GPU parity: batched quantized GEMM (bf16 activations, fp32 out) through the C ABI vs the fp64-accumulated oracle."""
import numpy as np
import pytest

from oracle import oracle_c, oracle_np
from skainet_amd import runtime, synth

pytestmark = pytest.mark.gpu
Q8_0, Q4_K, Q6_K = 8, 12, 14
TOL = 1e-3  # max |a - r| / max(|r|, 1e-3 * max|r|)


@pytest.mark.parametrize(
    "qtype,m,n,k",
    [
        (Q4_K, 512, 256, 4096),
        (Q6_K, 512, 256, 4096),
        (Q8_0, 64, 128, 1024),
        (Q4_K, 1, 64, 256),       # a single activation row
        (Q4_K, 33, 100, 768),     # ragged in m and n
        (Q6_K, 130, 65, 512),
        (Q4_K, 200, 192, 11008),  # the FFN-down row length (43 superblocks)
    ],
)
def test_gemm_vs_oracle(hip, qtype, m, n, k):
    raw = synth.weight(qtype, n, k, seed=3 * n + k + qtype)
    a = synth.activation_bf16((m, k), seed=m + 17)
    got = hip.gemm_q_host(qtype, raw, n, k, a, m)
    want = oracle_c.gemm_q(qtype, raw, n, k, a, m)
    err = oracle_np.rel_err(got, want)
    assert err <= TOL, f"rel err {err}"


@pytest.mark.parametrize("qtype", [Q4_K, Q6_K])
def test_gemm_rows_match_matvec(hip, qtype):
    m, n, k = 8, 128, 2048
    raw = synth.weight(qtype, n, k, seed=77)
    a = synth.activation_bf16((m, k), seed=78)
    c = hip.gemm_q_host(qtype, raw, n, k, a, m)
    af = oracle_np.bf16_to_f32(a).reshape(m, k)
    for r in range(m):
        y = hip.matvec_q_host(qtype, raw, n, k, af[r])
        assert oracle_np.rel_err(c[r], y) <= TOL


def test_gemm_large_activations_are_rescaled(hip):
    # rows far outside fp16 range (|a| up to ~1e6) and tiny rows must both come out right
    m, n, k = 4, 64, 1024
    raw = synth.weight(Q4_K, n, k, seed=5)
    x = np.random.default_rng(6).standard_normal((m, k)).astype(np.float32)
    x[0] *= 3.0e5
    x[1] *= 1.0e-3
    x[2, 17] = 9.0e5
    a = synth.f32_to_bf16_bits(x)
    got = hip.gemm_q_host(Q4_K, raw, n, k, a, m)
    want = oracle_c.gemm_q(Q4_K, raw, n, k, a, m)
    for r in range(m):
        assert oracle_np.rel_err(got[r], want[r]) <= TOL, r


@pytest.mark.parametrize("qtype", [Q4_K, Q6_K])
def test_gemm_extreme_rows(hip, qtype):
    """Rows the activation rescaling has to survive: all zero, a single non-zero element, the smallest bf16
    normals, a 2^40 dynamic range inside one row, negative-only and alternating signs."""
    m, n, k = 8, 96, 2048
    raw = synth.weight(qtype, n, k, seed=21)
    rng = np.random.default_rng(22)
    x = rng.standard_normal((m, k)).astype(np.float32)
    x[0] = 0.0
    x[1] = 0.0
    x[1, 1029] = -3.0
    x[2] *= 1.0e-30
    x[3] *= np.exp2(rng.integers(-20, 20, size=k)).astype(np.float32)
    x[4] = -np.abs(x[4])
    x[5] = np.where(np.arange(k) % 2 == 0, 1.0, -1.0)
    x[6] *= 6.0e4   # around the fp16 maximum before rescaling
    x[7, : k // 2] = 0.0
    a = synth.f32_to_bf16_bits(x)
    got = hip.gemm_q_host(qtype, raw, n, k, a, m)
    want = oracle_c.gemm_q(qtype, raw, n, k, a, m)
    assert np.all(got[0] == 0.0)
    w = oracle_c.dequant(qtype, raw).reshape(n, k)
    # a single non-zero activation returns a column of the weights: to 1e-6 of the column's largest magnitude
    # (a weight is the difference of two products, each of which is kept to about 2^-22)
    col = -3.0 * w[:, 1029]
    assert np.abs(got[1] - col).max() <= 1e-6 * np.abs(col).max(), np.abs(got[1] - col).max() / np.abs(col).max()
    for r in range(2, m):
        assert oracle_np.rel_err(got[r], want[r]) <= TOL, r


def test_gemm_q4k_superblock_scale_extremes(hip):
    """The Q4_K kernel keeps a column's accumulators in units of the current superblock's d: superblocks with
    d = 0, negative d or dmin, dmin = 0, d a subnormal, |dmin / d| from 2^-20 to 2^20, and d jumping by 2^20
    between neighbouring superblocks must all come out right."""
    m, n, k = 40, 64, 4096
    nb = k // 256
    raw = synth.weight(Q4_K, n, k, seed=91).reshape(n, nb, 144).copy()
    f16 = lambda v: np.array([v], dtype=np.float16).view(np.uint8)  # noqa: E731
    cases = [(0.0, 0.01), (0.0, 0.0), (-0.02, 0.01), (0.02, -0.01), (0.01, 0.0), (6e-8, 1e-7), (1e-5, 10.0),
             (1e-6, 1.0), (10.0, 1e-5), (500.0, 0.5), (3e-5, 0.03), (0.03, 3e-5), (-1e-4, -20.0), (2e-7, 0.2)]
    rng = np.random.default_rng(92)
    for col in range(n):
        for sb in range(nb):
            if col < 8 and sb % 3 == 1:
                continue  # a few ordinary superblocks in between
            d, dmin = cases[rng.integers(len(cases))] if col < 48 else cases[(col + sb) % len(cases)]
            raw[col, sb, 0:2] = f16(d)
            raw[col, sb, 2:4] = f16(dmin)
    raw[48] = raw[48, 0]  # every superblock the same
    raw[49, :, 0:2] = f16(0.0)  # a column with no live superblock at all
    raw = raw.reshape(-1)
    a = synth.activation_bf16((m, k), seed=93)
    got = hip.gemm_q_host(Q4_K, raw, n, k, a, m)
    want = oracle_c.gemm_q(Q4_K, raw, n, k, a, m)
    assert np.all(np.isfinite(got))
    for col in range(n):  # column by column: their magnitudes differ by many orders
        assert oracle_np.rel_err(got[:, col], want[:, col]) <= TOL, col


def test_gemm_q4k_several_row_tiles_and_ragged_columns(hip):
    """Three 128-row tiles (the last one partial) and a column count that is not a multiple of the 64-column tile."""
    m, n, k = 300, 200, 1280
    raw = synth.weight(Q4_K, n, k, seed=95)
    a = synth.activation_bf16((m, k), seed=96)
    got = hip.gemm_q_host(Q4_K, raw, n, k, a, m)
    want = oracle_c.gemm_q(Q4_K, raw, n, k, a, m)
    assert oracle_np.rel_err(got, want) <= TOL


@pytest.mark.parametrize(
    "m,n,k",
    [
        (1, 1, 64),       # one k-step per wavefront
        (32, 31, 192),    # fewer steps than the prefetch ring holds
        (33, 65, 320),    # two row blocks, a second column tile of one column
        (64, 100, 448),
        (65, 64, 1088),   # the smallest shape on 128-row tiles; steps not a multiple of the ring depth
        (129, 130, 2112),
        (260, 96, 6400),
    ],
)
def test_gemm_general_path_shapes(hip, m, n, k):
    """Row counts on every tile height (32, 64, 128 rows), ragged columns, and row lengths whose k-steps per
    wavefront are below, at and off multiples of the kernel's prefetch depth (Q8_0: k a multiple of 64)."""
    raw = synth.weight(Q8_0, n, k, seed=n + k)
    a = synth.activation_bf16((m, k), seed=m + k)
    got = hip.gemm_q_host(Q8_0, raw, n, k, a, m)
    want = oracle_c.gemm_q(Q8_0, raw, n, k, a, m)
    assert oracle_np.rel_err(got, want) <= TOL


def test_gemm_general_path_weight_magnitudes(hip):
    """Dense fp32 weights from 1e-4 to 4e4 (rows of one magnitude each, and rows mixing them): the fp16 pair the
    kernel multiplies with keeps a weight to 2^-22 relative or 2^-36 absolute, whichever is larger -- the same
    precision from fp16's subnormal range to its largest finite value."""
    F32 = 0
    m, n, k = 48, 96, 1024
    rng = np.random.default_rng(31)
    w = rng.standard_normal((n, k)).astype(np.float32)
    scales = np.array([3e-4, 1e-3, 0.02, 1.0, 37.0, 2.0e3, 4.0e4], dtype=np.float32)
    for r in range(n):
        if r < 64:
            w[r] *= scales[r % len(scales)] / 4.0  # (|N(0,1)| stays below 6 here: nothing overflows fp16)
        else:
            w[r] *= scales[rng.integers(len(scales) - 1, size=k)]
    a = synth.activation_bf16((m, k), seed=32)
    got = hip.gemm_q_host(F32, w.view(np.uint8).reshape(-1), n, k, a, m)
    want = oracle_c.gemm_q(F32, w.view(np.uint8).reshape(-1), n, k, a, m)
    assert np.all(np.isfinite(got))
    for col in range(n):  # column by column: their magnitudes differ by many orders
        assert oracle_np.rel_err(got[:, col], want[:, col]) <= TOL, col


@pytest.mark.parametrize("m,n,k", [(512, 256, 4096), (200, 192, 11008), (130, 100, 768), (65, 64, 256), (300, 129, 1024), (1, 1, 256)])
def test_gemm_q4k_wide_tile_kernel_on_small_and_ragged_shapes(hip, m, n, k):
    """The Q4_K kernel with 256 x 128 tiles, which the library picks by itself only where such tiles fill the machine
    (N = 14336 at M = 512: test_gemm_benchmark_shape_q4k_n14336), forced on shapes with partial tiles in both
    directions and with 1, 3, 4, 16 and 43 superblocks per row."""
    raw = synth.weight(Q4_K, n, k, seed=3 * n + k)
    a = synth.activation_bf16((m, k), seed=m + 17)
    want = oracle_c.gemm_q(Q4_K, raw, n, k, a, m)
    hip.set_option("gemm.tile", 3)
    try:
        got = hip.gemm_q_host(Q4_K, raw, n, k, a, m)
    finally:
        hip.set_option("gemm.tile", 0)
    err = oracle_np.rel_err(got, want)
    assert err <= TOL, f"rel err {err}"


@pytest.mark.parametrize("m,n,k", [(160, 100, 1280), (40, 64, 256), (512, 64, 2048), (300, 200, 768)])
def test_gemm_q6k_full_range_of_the_block_fields(hip, m, n, k):
    """Q6_K blocks as real files hold them: int8 scales over all of -128..127 (the benchmark's generator stops at
    +-32), d of either sign, zero and subnormal d, superblock counts that do not divide by the four wavefronts that
    share a tile's k; with every form of the kernels that unpack the blocks themselves (128 x 64 or 256 x 128 tiles,
    specialised wavefronts or not) and without them."""
    rng = np.random.default_rng(1000 + k)
    raw = synth.weight(Q6_K, n, k, seed=31).reshape(-1, 210).copy()
    nblk = raw.shape[0]
    raw[:, 192:208] = rng.integers(-128, 128, size=(nblk, 16), dtype=np.int8).view(np.uint8)
    raw[::7, 192:208] = np.array([-128, 127, -1, 0, 15, 16, -16, -17] * 2, dtype=np.int8).view(np.uint8)
    d = (rng.standard_normal(nblk) * 0.01).astype(np.float16)
    d[::5] = 0.0
    d[3::11] = np.float16(6e-8)  # the smallest subnormal
    raw[:, 208:210] = d.view(np.uint8).reshape(-1, 2)
    raw = raw.reshape(-1)
    a = synth.activation_bf16((m, k), seed=m + 5)
    want = oracle_c.gemm_q(Q6_K, raw, n, k, a, m)
    for fused, tile in ((1, 0), (1, 3), (2, 0), (0, 0)):  # (tile 3: the 256 x 128 form, otherwise for wide matrices only)
        hip.set_option("gemm.q6k_fused", fused)
        hip.set_option("gemm.tile", tile)
        try:
            got = hip.gemm_q_host(Q6_K, raw, n, k, a, m)
        finally:
            hip.set_option("gemm.q6k_fused", 1)
            hip.set_option("gemm.tile", 0)
        err = oracle_np.rel_err(got, want)
        assert err <= TOL, f"fused={fused} tile={tile}: rel err {err}"


@pytest.mark.parametrize("n", [4096, 14336])
def test_gemm_benchmark_shapes_q6k(hip, n):
    """M=512, K=4096 with Q6_K weights (the mixed-precision prefill case), sampled columns."""
    m, k = 512, 4096
    raw = synth.weight(Q6_K, n, k, seed=11)
    a = synth.activation_bf16((m, k), seed=12)
    got = hip.gemm_q_host(Q6_K, raw, n, k, a, m)
    rows = np.arange(0, n, 127)
    rb = raw.reshape(n, -1)[rows].reshape(-1)
    want = oracle_c.gemm_q(Q6_K, rb, len(rows), k, a, m)
    floor = 1e-3 * np.abs(got).max()
    err = np.max(np.abs(got[:, rows] - want) / np.maximum(np.abs(want), floor))
    assert err <= TOL, err


def test_gemm_benchmark_shape_q4k_n14336(hip):
    """M=512, K=4096, N=14336 with Q4_K weights: the wide cell of the mixed Q4_K/Q6_K prefill case, sampled columns."""
    m, n, k = 512, 14336, 4096
    raw = synth.weight(Q4_K, n, k, seed=13)
    a = synth.activation_bf16((m, k), seed=14)
    got = hip.gemm_q_host(Q4_K, raw, n, k, a, m)
    rows = np.arange(0, n, 127)
    rb = raw.reshape(n, -1)[rows].reshape(-1)
    want = oracle_c.gemm_q(Q4_K, rb, len(rows), k, a, m)
    floor = 1e-3 * np.abs(got).max()
    err = np.max(np.abs(got[:, rows] - want) / np.maximum(np.abs(want), floor))
    assert err <= TOL, err


@pytest.mark.parametrize("t", [Q4_K, Q6_K])
def test_gemm_2000_rows_take_the_wide_tile_kernels_by_themselves(hip, t):
    """M = 2000, N = 4096, K = 2048: eight row tiles x 32 column tiles of 256 x 128 fill the 256 compute units, so the
    library picks the wide-tile kernels without being told; the last row tile has 208 rows.  Sampled columns."""
    m, n, k = 2000, 4096, 2048
    raw = synth.weight(t, n, k, seed=23)
    a = synth.activation_bf16((m, k), seed=24)
    got = hip.gemm_q_host(t, raw, n, k, a, m)
    rows = np.arange(0, n, 61)
    rb = raw.reshape(n, -1)[rows].reshape(-1)
    want = oracle_c.gemm_q(t, rb, len(rows), k, a, m)
    floor = 1e-3 * np.abs(got).max()
    err = np.max(np.abs(got[:, rows] - want) / np.maximum(np.abs(want), floor))
    assert err <= TOL, err


def test_gemm_full_width_slice(hip):
    """The benchmark shape M=512, K=4096 at N=4096: checked on a strided sample of the oracle's columns."""
    m, n, k = 512, 4096, 4096
    raw = synth.weight(Q4_K, n, k, seed=9)
    a = synth.activation_bf16((m, k), seed=10)
    got = hip.gemm_q_host(Q4_K, raw, n, k, a, m)
    rows = np.arange(0, n, 61)
    rb = raw.reshape(n, -1)[rows].reshape(-1)
    want = oracle_c.gemm_q(Q4_K, rb, len(rows), k, a, m)
    # normalise with the whole output's scale, as the metric is defined over the full result
    floor = 1e-3 * np.abs(got).max()
    err = np.max(np.abs(got[:, rows] - want) / np.maximum(np.abs(want), floor))
    assert err <= TOL, err


@pytest.mark.parametrize("qtype", [Q6_K, synth.Q8_0, synth.Q5_K, synth.Q4_0, Q4_K])
@pytest.mark.parametrize("m,n,k", [(512, 320, 1024), (40, 100, 512), (3, 64, 256)])
def test_gemm_with_expanded_weights_equals_the_per_call_path(hip, qtype, m, n, k):
    """skn_gemm_expand + skn_gemm_expanded: the weight pass of the general path done once; same kernels, so the
    product equals skn_gemm_q's bit for bit for every other format, and the oracle's to the tolerance (also for Q4_K,
    which skn_gemm_q multiplies on its own path, as it does Q6_K unless the option gemm.q6k_fused is off: another order
    of additions, so its bits are compared with the option off).  The copy serves any number of products."""
    raw = synth.weight(qtype, n, k, seed=21)
    w = hip.to_device(raw)
    assert hip.gemm_expanded_bytes(qtype, n, k) == (n + 63) // 64 * 64 * k * 4
    exp = hip.gemm_expand(qtype, w, n, k)
    for seed in (22, 23):
        a = synth.activation_bf16((m, k), seed=seed)
        a_dev = hip.to_device(a)
        c = hip.alloc(4 * m * n)
        hip.memset(c, 0xFF, 4 * m * n)
        hip.gemm_expanded(exp, n, k, a_dev, m, c)
        got = c.download(np.float32, m * n).reshape(m, n)
        assert oracle_np.rel_err(got, oracle_c.gemm_q(qtype, raw, n, k, a, m)) <= TOL
        if qtype != Q4_K:
            hip.set_option("gemm.q6k_fused", 0)
            try:
                per_call = hip.gemm_q_host(qtype, raw, n, k, a, m)
            finally:
                hip.set_option("gemm.q6k_fused", 1)
            assert np.array_equal(got.view(np.uint32), per_call.view(np.uint32))
        a_dev.free(), c.free()
    exp.free(), w.free()


def test_gemm_expanded_benchmark_shape_q6k(hip):
    """M=512, K=4096, N=4096 with Q6_K weights through the kept copy, sampled columns."""
    m, n, k = 512, 4096, 4096
    raw = synth.weight(Q6_K, n, k, seed=11)
    a = synth.activation_bf16((m, k), seed=12)
    w, a_dev, c = hip.to_device(raw), hip.to_device(a), hip.alloc(4 * m * n)
    exp = hip.gemm_expand(Q6_K, w, n, k)
    hip.gemm_expanded(exp, n, k, a_dev, m, c)
    got = c.download(np.float32, m * n).reshape(m, n)
    rows = np.arange(0, n, 127)
    want = oracle_c.gemm_q(Q6_K, raw.reshape(n, -1)[rows].reshape(-1), len(rows), k, a, m)
    err = np.max(np.abs(got[:, rows] - want) / np.maximum(np.abs(want), 1e-3 * np.abs(got).max()))
    assert err <= TOL, err
    for b in (w, a_dev, c, exp):
        b.free()


def test_gemm_expanded_errors(hip):
    buf = hip.alloc(1 << 16)
    with pytest.raises(runtime.SknError, match="not a multiple of block size"):
        hip.gemm_expanded_bytes(Q6_K, 4, 100)
    with pytest.raises(runtime.SknError, match="multiple of 64"):
        hip.gemm_expanded_bytes(synth.Q8_0, 4, 96)
    with pytest.raises(runtime.SknError, match="not supported"):
        hip.gemm_expanded_bytes(999, 4, 256)
    with pytest.raises(runtime.SknError, match="null pointer"):
        hip._check(hip.lib.skn_gemm_expand(hip.handle, Q6_K, None, 4, 256, runtime._ptr(buf)))
    with pytest.raises(runtime.SknError, match="multiple of 64"):
        hip.gemm_expanded(buf, 4, 96, buf, 2, buf)
    assert hip.gemm_expanded_bytes(Q6_K, 0, 256) == 0
    hip.gemm_expanded(buf, 0, 256, buf, 2, buf)  # nothing to do
    buf.free()
