"""skn_synth_* (the library's seeded generators, host side) against their NumPy restatement in skainet_amd/synth.py:
byte for byte, at ragged sizes, plus the statistics BASELINE's recipe states and checksums a C client checks too.
CPU only: these entry points touch no device."""
import numpy as np
import pytest

from oracle import oracle_c
from skainet_amd import runtime, synth

Q8_0, Q4_K, Q6_K = 8, 12, 14


@pytest.mark.parametrize("qtype", [Q8_0, Q4_K, Q6_K])
@pytest.mark.parametrize("rows,k,seed", [(1, 256, 0), (3, 512, 1), (17, 2304, 2**63 + 5), (64, 4096, 123456789), (0, 256, 9)])
def test_library_weights_equal_the_numpy_restatement(qtype, rows, k, seed):
    got = runtime.synth_weight(qtype, rows, k, seed)
    want = synth.lib_weight(qtype, rows, k, seed)
    assert got.dtype == np.uint8 and got.size == rows * runtime.row_bytes(qtype, k)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("n,seed", [(0, 1), (1, 1), (7, 2), (4096, 3), (11008, 2**64 - 1)])
def test_library_vectors_equal_the_numpy_restatement(n, seed):
    assert np.array_equal(runtime.synth_activation_f32(n, seed).view(np.uint32), synth.lib_activation_f32(n, seed).view(np.uint32))
    assert np.array_equal(runtime.synth_activation_bf16(n, seed), synth.lib_activation_bf16(n, seed))
    assert np.array_equal(runtime.synth_kv_f16(n, seed), synth.lib_kv_f16(n, seed))


def test_fp16_conversion_of_the_library_over_its_whole_range():
    """The generators convert through their own fp32 -> fp16 routine: scaled draws reach fp16 subnormals (|N| * 0.005
    below 6.1e-5) and every exponent up to 6; all must equal NumPy's round-to-nearest-even."""
    n = 200000
    raw = runtime.synth_weight(Q4_K, n // 8, 2048, 77).reshape(-1, 144)
    want = synth.lib_weight(Q4_K, n // 8, 2048, 77).reshape(-1, 144)
    d = raw[:, 0:4].copy().view(np.float16).astype(np.float32)
    assert np.array_equal(raw[:, 0:4], want[:, 0:4])
    assert (d[:, 1] < 6.1e-5).sum() > 100 and (d[:, 1] > 6.1e-5).sum() > 100  # subnormal and normal dmin both occur


def test_statistics_follow_the_recipe():
    """d = |N| * 0.02 / 0.01 / 0.005 (mean |N| = 0.798), quants uniform over their ranges, values of unit variance."""
    x = synth.lib_activation_f32(200000, 5).astype(np.float64)
    assert abs(x.mean()) < 0.01 and abs(x.std() - 1.0) < 0.01 and np.abs(x).max() <= 6.0
    q8 = runtime.synth_weight(Q8_0, 64, 4096, 11).reshape(-1, 34)
    assert abs(q8[:, 0:2].copy().view(np.float16).astype(np.float64).mean() / (0.798 * 0.02) - 1) < 0.05
    q = q8[:, 2:].view(np.int8)
    assert q.min() == -127 and q.max() == 127 and abs(q.astype(np.float64).mean()) < 0.5
    q4 = runtime.synth_weight(Q4_K, 64, 4096, 12).reshape(-1, 144)
    h = q4[:, 0:4].copy().view(np.float16).astype(np.float64)
    assert abs(h[:, 0].mean() / (0.798 * 0.01) - 1) < 0.08 and abs(h[:, 1].mean() / (0.798 * 0.005) - 1) < 0.08
    w = oracle_c.dequant(Q4_K, q4.reshape(-1))
    assert np.isfinite(w).all()
    nib = np.bincount(np.concatenate([q4[:, 16:].reshape(-1) & 15, q4[:, 16:].reshape(-1) >> 4]), minlength=16)
    assert nib.min() > 0.9 * nib.mean()
    q6 = runtime.synth_weight(Q6_K, 64, 4096, 13).reshape(-1, 210)
    sc = q6[:, 192:208].view(np.int8)
    assert sc.min() == -32 and sc.max() == 31
    assert np.isfinite(oracle_c.dequant(Q6_K, q6.reshape(-1))).all()


def test_checksums_known_to_the_c_client():
    """The same constants stand in tests/c/abi_client.c: a C harness and this one see the same buffers."""
    w = runtime.synth_weight(Q4_K, 2, 512, 42)
    assert runtime.synth_checksum(w) == synth.lib_checksum(w)
    assert runtime.synth_checksum(w) == CHECKSUM_Q4K_2x512_SEED42
    x = runtime.synth_activation_f32(512, 42)
    assert runtime.synth_checksum(x) == synth.lib_checksum(x) == CHECKSUM_F32_512_SEED42


def test_argument_errors():
    with pytest.raises(runtime.SknError) as e:
        runtime.synth_weight(2, 1, 256, 0)  # Q4_0 has no generator
    assert e.value.code == runtime.ERR_TYPE
    lib = runtime.load_library()
    buf = np.empty(10, dtype=np.uint8)
    assert lib.skn_synth_weight(Q4_K, 1, 100, 0, buf.ctypes.data, 10) == runtime.ERR_SHAPE
    assert b"not a multiple of block size (256)" in lib.skn_last_error(None)
    assert lib.skn_synth_weight(Q4_K, 1, 256, 0, buf.ctypes.data, 10) == runtime.ERR_SHAPE
    assert lib.skn_synth_activation_f32(-1, 0, None) == runtime.ERR_ARG


CHECKSUM_Q4K_2x512_SEED42 = 0xB1D64B923C1648B4
CHECKSUM_F32_512_SEED42 = 0x9A9CFB33CCC7FEA4
