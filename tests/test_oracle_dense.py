"""CPU: dense matmul / Linear semantics of the oracles against the known answers the reference's tests hold,
and the quantized matvec / GEMM oracles against their reduction to that dense semantics."""
import json
import math
import os

import numpy as np
import pytest

from oracle import oracle_c, oracle_np
from skainet_amd import synth

Q8_0, Q4_K, Q6_K = 8, 12, 14


@pytest.fixture(scope="module")
def cases(golden_dir):
    with open(os.path.join(golden_dir, "tensor_test_vectors.json")) as f:
        return json.load(f)["cases"]


def _t(case, i):
    t = case["tensors"][i]
    return np.array(t["values"], dtype=np.float64).reshape(t["shape"] or [-1])


def test_vector_matrix_known_answers(cases):
    # reference TensorTest.kt:39-53
    for name in ("matmulOfVectorAndMatrix", "matmulOfVectorSingleAndMatrix"):
        c = cases[name]
        x, b = _t(c, 0), _t(c, 1)
        assert oracle_c.dense_vecmat(x, b).tolist() == c["expected"]
        assert oracle_np.dense_vecmat(x, b).tolist() == c["expected"]


def test_matrix_matrix_known_answer_and_shape_error(cases):
    # reference TensorTest.kt:56-70
    c = cases["matmulOfMatrixAndMatrix"]
    assert oracle_c.dense_matmul(_t(c, 0), _t(c, 1)).reshape(-1).tolist() == c["expected"]
    assert oracle_np.dense_matmul(_t(c, 0), _t(c, 1)).reshape(-1).tolist() == c["expected"]
    bad = cases["matmulOfMatrixAndMatrixWithWrongShaoe"]
    assert bad["error"] == "Shapes do not align."
    with pytest.raises(ValueError, match="Shapes do not align."):
        oracle_np.dense_matmul(_t(bad, 0), _t(bad, 1))


def test_1x16_times_16x16(cases):
    # reference TensorTest.kt:72-391: expected row within 1e-4
    c = cases["matmul 1x16  16x16"]
    a, b, want = _t(c, 0), _t(c, 1), _t(c, 2)
    assert a.shape == (1, 16) and b.shape == (16, 16) and want.shape == (1, 16)
    assert np.max(np.abs(oracle_c.dense_matmul(a, b) - want)) < 1e-4
    assert np.max(np.abs(oracle_c.dense_vecmat(a[0], b) - want[0])) < 1e-4
    assert np.max(np.abs(oracle_np.dense_matmul(a, b) - want)) < 1e-4


def test_3d_times_2d_rows(cases):
    # reference TensorTest.kt:472-538: every [.., width] row times the [width, out] matrix
    c = cases["matmulOf3DTensorAnd2DMatrix"]
    x, w = _t(c, 0), _t(c, 1)
    got = oracle_c.dense_matmul(x.reshape(-1, x.shape[-1]), w).reshape(-1)
    want = np.array(c["expected"])
    assert np.max(np.abs(got[: want.size] - want)) < 1e-10


def test_sine_mlp_end_to_end(golden_dir):
    # reference io/src/jvmTest/.../CsvParametersLoaderTest.kt:33-72: |mlp(pi/2) - 1| < 0.01 through three Linear layers
    with open(os.path.join(golden_dir, "sinus-approximator.json")) as f:
        params = {e["unique_parameter_name"]: np.array(e["tensor"]["values"]).reshape(e["tensor"]["shape"]) for e in json.load(f)}
    assert len(params) == 6
    x = np.array([math.pi / 2.0])
    for i, last in ((1, False), (3, False), (5, True)):
        x = oracle_np.linear(x, params[f"linear-{i}.weight"], params[f"linear-{i}.bias"])
        if not last:
            x = np.maximum(x, 0.0)
    assert abs(x[0] - 1.0) < 0.01


@pytest.mark.parametrize("qtype", [Q8_0, Q4_K, Q6_K])
def test_quantized_matvec_reduces_to_dense_reference(qtype):
    n, k = 24, 1024
    raw = synth.weight(qtype, n, k, seed=21 + qtype)
    x = synth.activation_f32(k, seed=5)
    w = oracle_np.dequant(qtype, raw).reshape(n, k).astype(np.float64)
    # Linear.kt:48 semantics: x.matmul(W.t()) through the reference's vec x mat loop
    want = oracle_c.dense_vecmat(x.astype(np.float64), np.ascontiguousarray(w.T))
    got_c = oracle_c.matvec_q(qtype, raw, n, k, x)
    got_np = oracle_np.matvec_q(qtype, raw, n, k, x)
    got_ref_alg = oracle_c.matvec_q(qtype, raw, n, k, x, reference_algorithm=True)
    assert oracle_np.rel_err(got_c, want) < 1e-6
    assert oracle_np.rel_err(got_np, want) < 1e-6
    assert np.array_equal(got_ref_alg, want.astype(np.float32))
    # one-hot activation picks out a column of deq(W) exactly
    e = np.zeros(k, dtype=np.float32)
    e[517] = 1.0
    assert np.array_equal(oracle_c.matvec_q(qtype, raw, n, k, e), w[:, 517].astype(np.float32))
    # linearity in x
    x2 = synth.activation_f32(k, seed=6)
    lhs = oracle_c.matvec_q(qtype, raw, n, k, (x + x2).astype(np.float32)).astype(np.float64)
    rhs = got_c.astype(np.float64) + oracle_c.matvec_q(qtype, raw, n, k, x2)
    assert oracle_np.rel_err(lhs, rhs) < 1e-5


@pytest.mark.parametrize("qtype", [Q4_K, Q6_K])
def test_quantized_gemm_reduces_to_dense_reference(qtype):
    n, k, m = 16, 512, 5
    raw = synth.weight(qtype, n, k, seed=31 + qtype)
    a = synth.activation_bf16((m, k), seed=8)
    w = oracle_np.dequant(qtype, raw).reshape(n, k).astype(np.float64)
    af = oracle_np.bf16_to_f32(a).astype(np.float64)
    want = oracle_c.dense_matmul(af, np.ascontiguousarray(w.T))
    got = oracle_c.gemm_q(qtype, raw, n, k, a, m)
    assert oracle_np.rel_err(got, want) < 1e-6
    assert oracle_np.rel_err(oracle_np.gemm_q(qtype, raw, n, k, a, m), want) < 1e-6
    # row m of the GEMM is the matvec on activation row m
    for r in range(m):
        mv = oracle_c.matvec_q(qtype, raw, n, k, af[r].astype(np.float32))
        assert oracle_np.rel_err(got[r], mv) < 1e-6


def test_matvec_shape_errors():
    raw = synth.weight(Q4_K, 2, 256, seed=1)
    with pytest.raises(ValueError):
        oracle_c.matvec_q(Q4_K, raw, 2, 200, np.zeros(200, dtype=np.float32))
    with pytest.raises(ValueError):
        oracle_np.matvec_q(Q4_K, raw, 2, 200, np.zeros(200, dtype=np.float32))


def test_bf16_conversion_round_trip():
    x = np.random.default_rng(3).standard_normal(10000).astype(np.float32)
    bits = synth.f32_to_bf16_bits(x)
    assert np.array_equal(bits, oracle_np.f32_to_bf16(x))
    back = oracle_np.bf16_to_f32(bits)
    assert np.max(np.abs(back - x) / np.abs(x)) <= 2.0 ** -8
    assert np.array_equal(oracle_np.f32_to_bf16(back), bits)
