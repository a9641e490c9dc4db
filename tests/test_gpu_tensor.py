"""GPU: the reference-shaped tensor wrappers (QuantizedTensor / DeviceTensor / QuantizedLinear) and a GGUF file
loaded to the device end to end.  The known answers are the reference's own TensorTest matmul cases, carried
through Q8_0 weights that represent them exactly."""
import json
import math
import os

import numpy as np
import pytest

from oracle import oracle_c, oracle_np
from skainet_amd import gguf, synth
from skainet_amd.tensor import MLP, DeviceTensor, QuantizedLinear, QuantizedTensor, ReLU, Shape

pytestmark = pytest.mark.gpu


def _q8_exact(rows):
    """[n, k<=32-multiple] small-integer matrix -> Q8_0 bytes holding it exactly (d = 1)."""
    rows = np.asarray(rows)
    n, k = rows.shape
    kp = -(-k // 32) * 32
    q = np.zeros((n, kp), dtype=np.int8)
    q[:, :k] = rows
    blocks = np.zeros((n, kp // 32, 34), dtype=np.uint8)
    blocks[:, :, 0:2] = np.array([1.0], dtype=np.float16).view(np.uint8)
    blocks[:, :, 2:] = q.reshape(n, kp // 32, 32).view(np.uint8)
    return blocks.reshape(-1), kp


def test_reference_matmul_known_answers_through_quantized_weights(hip, golden_dir):
    cases = json.load(open(os.path.join(golden_dir, "tensor_test_vectors.json")))["cases"]
    # TensorTest.kt:39-45: [1,2] . [[1,2,3],[4,5,6]] = [9,12,15]; as Linear: W = B^T is [out=3, in=2]
    c = cases["matmulOfVectorAndMatrix"]
    x = np.array(c["tensors"][0]["values"])
    b = np.array(c["tensors"][1]["values"]).reshape(c["tensors"][1]["shape"])
    raw, kp = _q8_exact(b.T)
    w = QuantizedTensor.from_bytes(hip, synth.Q8_0, 3, kp, raw)
    xp = np.zeros(kp, dtype=np.float32)
    xp[: x.size] = x
    y = DeviceTensor.from_numpy(hip, xp).matmul(w.t())
    assert y.shape == Shape(3) and y.numpy().tolist() == c["expected"]
    # TensorTest.kt:56-62: the rank-2 case through the GEMM path (k padded to the GEMM's 64-element granule)
    c = cases["matmulOfMatrixAndMatrix"]
    a = np.array(c["tensors"][0]["values"]).reshape(2, 3)
    b = np.array(c["tensors"][1]["values"]).reshape(3, 2)
    bt = np.zeros((2, 64))
    bt[:, :3] = b.T
    raw, kp = _q8_exact(bt)
    w = QuantizedTensor.from_bytes(hip, synth.Q8_0, 2, kp, raw)
    ap = np.zeros((2, kp), dtype=np.float32)
    ap[:, :3] = a
    got = DeviceTensor.from_numpy(hip, ap).matmul(w.t())
    assert got.shape == Shape(2, 2) and got.numpy().reshape(-1).tolist() == c["expected"]


@pytest.mark.parametrize("case", ["matmulOf3DTensorAnd2DMatrix", "matmulOf4DNCHWTensorAnd2DMatrix"])
def test_reference_3d_and_4d_inputs_through_the_gemm(hip, golden_dir, case):
    """TensorTest.kt:393-538: a [3, 2, 4] and a [2, 3, 2, 4] tensor times a [4, 3] matrix -- every row of four times
    the matrix, the leading dimensions kept.  The rows are small integers (exact in the bf16 the GEMM rounds them to),
    the matrix 0.1 .. 1.2 as dense F32 weights W = B^T (k padded to the GEMM's 64-element granule): the reference's
    expected values (it lists the first 18) to fp32 accuracy."""
    c = json.load(open(os.path.join(golden_dir, "tensor_test_vectors.json")))["cases"][case]
    x = np.array(c["tensors"][0]["values"]).reshape(c["tensors"][0]["shape"])
    b = np.array(c["tensors"][1]["values"]).reshape(c["tensors"][1]["shape"])
    kp = 64
    wt = np.zeros((b.shape[1], kp), dtype=np.float32)
    wt[:, : b.shape[0]] = b.T
    w = QuantizedTensor.from_bytes(hip, synth.F32, b.shape[1], kp, wt.view(np.uint8))
    xp = np.zeros(x.shape[:-1] + (kp,), dtype=np.float32)
    xp[..., : x.shape[-1]] = x
    got = DeviceTensor.from_numpy(hip, xp).matmul(w.t())
    assert got.shape == Shape(*x.shape[:-1], b.shape[1])
    want = np.array(c["expected"], dtype=np.float64)
    flat = got.numpy().reshape(-1).astype(np.float64)
    assert np.max(np.abs(flat[: want.size] - want) / np.abs(want)) < 1e-6
    assert np.max(np.abs(flat - (x @ b).reshape(-1)) / np.abs((x @ b).reshape(-1))) < 1e-6
    with pytest.raises(ValueError, match="Shapes do not align"):
        DeviceTensor.from_numpy(hip, xp[..., :32]).matmul(w.t())


def test_reference_1x16_times_16x16_through_the_matvec(hip, golden_dir):
    """TensorTest.kt:72-391: the 1x16 row times the 16x16 matrix, expected row within 1e-4 -- as Linear computes it,
    x.matmul(W.t()) with W = B^T held as dense F32 rows on the device."""
    c = json.load(open(os.path.join(golden_dir, "tensor_test_vectors.json")))["cases"]["matmul 1x16  16x16"]
    a, b, want = (np.array(t["values"], dtype=np.float64).reshape(t["shape"]) for t in c["tensors"])
    assert a.shape == (1, 16) and b.shape == (16, 16) and want.shape == (1, 16)
    wt = np.ascontiguousarray(b.T, dtype=np.float32)  # [out, in]
    w = QuantizedTensor.from_bytes(hip, synth.F32, 16, 16, wt.view(np.uint8))
    y = DeviceTensor.from_numpy(hip, a[0]).matmul(w.t())
    assert y.shape == Shape(16)
    assert np.max(np.abs(y.numpy().astype(np.float64) - want[0])) < 1e-4


def test_sine_mlp_end_to_end_on_the_device(hip, golden_dir):
    """CsvParametersLoaderTest.kt:33-72: the 1-16-16-1 sine approximator (three Linear layers with bias, ReLU after
    the first two) loaded from the reference's own parameter file, |mlp(pi/2) - sin(pi/2)| < 0.01 -- every layer a
    QuantizedLinear over dense F32 rows on the device, the ReLUs device kernels, composed by the MLP container."""
    with open(os.path.join(golden_dir, "sinus-approximator.json")) as f:
        params = {e["unique_parameter_name"]: np.array(e["tensor"]["values"], dtype=np.float32).reshape(e["tensor"]["shape"])
                  for e in json.load(f)}
    assert len(params) == 6
    mods = []
    for i, last in ((1, False), (3, False), (5, True)):
        w, b = params[f"linear-{i}.weight"], params[f"linear-{i}.bias"]
        n_out, n_in = w.shape
        qt = QuantizedTensor.from_bytes(hip, synth.F32, n_out, n_in, np.ascontiguousarray(w).view(np.uint8))
        mods.append(QuantizedLinear(qt, DeviceTensor.from_numpy(hip, b), name=f"linear-{i}"))
        if not last:
            mods.append(ReLU())
    net = MLP(*mods)
    for angle in (math.pi / 2.0, 0.3, 1.0):
        x = DeviceTensor.from_numpy(hip, np.array([angle]))
        y = net(x).numpy()
        # the same stack on the oracle (fp64): the device result follows it to fp32 rounding
        r = np.array([angle])
        for i, last in ((1, False), (3, False), (5, True)):
            r = oracle_np.linear(r, params[f"linear-{i}.weight"].astype(np.float64), params[f"linear-{i}.bias"].astype(np.float64))
            if not last:
                r = np.maximum(r, 0.0)
        assert y.shape == (1,) and abs(float(y[0]) - float(r[0])) < 1e-5
    assert abs(float(net(DeviceTensor.from_numpy(hip, np.array([math.pi / 2.0]))).numpy()[0]) - 1.0) < 0.01


def test_relu_follows_the_reference(hip):
    x = np.array([-1.5, 0.0, -0.0, 2.25, np.nan, np.inf, -np.inf, 1e-38], dtype=np.float32)
    got = DeviceTensor.from_numpy(hip, x).relu().numpy()
    assert got.tolist() == [0.0, 0.0, 0.0, 2.25, 0.0, np.inf, 0.0, float(np.float32(1e-38))]


def test_shape_errors_follow_the_reference(hip):
    w = QuantizedTensor.from_bytes(hip, synth.Q4_K, 4, 256, synth.weight(synth.Q4_K, 4, 256, seed=1))
    x = DeviceTensor.from_numpy(hip, np.zeros(512, dtype=np.float32))
    with pytest.raises(ValueError, match="Shapes do not align."):  # TensorTest.kt:65-70
        x.matmul(w.t())
    with pytest.raises(ValueError, match="Unsupported tensor shapes for multiplication"):
        x.matmul(w)  # not transposed: [512] x [4, 256] is no Linear
    with pytest.raises(ValueError, match="Unsupported tensor shapes for multiplication"):
        w.matmul(x)
    assert w.t().shape == Shape(256, 4) and w.t().t().shape == Shape(4, 256) and w.t().buf is w.buf
    with pytest.raises(Exception, match="not a multiple of block size"):
        QuantizedTensor(hip, synth.Q4_K, Shape(4, 200), w.buf)


def test_quantized_linear_with_bias_and_dequantize(hip):
    n, k = 48, 1024
    raw = synth.weight(synth.Q6_K, n, k, seed=4)
    w = QuantizedTensor.from_bytes(hip, synth.Q6_K, n, k, raw)
    bias = np.random.default_rng(1).standard_normal(n).astype(np.float32)
    lin = QuantizedLinear(w, DeviceTensor.from_numpy(hip, bias))
    x = synth.activation_f32(k, seed=2)
    y = lin(DeviceTensor.from_numpy(hip, x)).numpy()
    want = oracle_c.matvec_q(synth.Q6_K, raw, n, k, x).astype(np.float64) + bias
    assert oracle_np.rel_err(y, want) <= 1e-3
    xs = np.random.default_rng(3).standard_normal((5, k)).astype(np.float32)
    ys = lin(DeviceTensor.from_numpy(hip, xs)).numpy()
    want = oracle_c.gemm_q(synth.Q6_K, raw, n, k, synth.f32_to_bf16_bits(xs), 5).astype(np.float64) + bias
    assert oracle_np.rel_err(ys, want) <= 1e-3
    deq = w.dequantize().numpy()
    assert np.array_equal(deq.view(np.uint32), oracle_c.dequant(synth.Q6_K, raw).reshape(n, k).view(np.uint32))


def test_gguf_file_to_device(hip, tmp_path):
    path = str(tmp_path / "m.gguf")
    n, k = 32, 512
    raw = synth.weight(synth.Q4_K, n, k, seed=9)
    gguf.write_gguf(path, {"general.architecture": "llama"}, [("blk.0.ffn_up.weight", 12, (n, k), raw)])
    r = gguf.GGUFReader(path)
    t = r.tensor("blk.0.ffn_up.weight")
    w = QuantizedTensor.from_bytes(hip, t.tensor_type, t.shape[0], t.shape[1], t.data)
    x = synth.activation_f32(k, seed=10)
    y = DeviceTensor.from_numpy(hip, x).matmul(w.t()).numpy()
    assert oracle_np.rel_err(y, oracle_c.matvec_q(12, raw, n, k, x)) <= 1e-3
    del t
    r.close()
