"""CPU: the GGUF reader against the reference's own fixture and against files written by write_gguf."""
import os
import struct

import numpy as np
import pytest

from oracle import oracle_np
from skainet_amd import gguf, synth


def test_reference_fixture(golden_dir):
    # gguf/src/jvmTest/resources/test_experiment.gguf: GGUF v3, three KV strings, three 3x3 F32 tensors, result = x + y
    r = gguf.GGUFReader(os.path.join(golden_dir, "test_experiment.gguf"))
    assert r.version == 3 and r.alignment == 32 and r.data_offset == 320
    assert r.fields["general.architecture"] == "llama"
    assert r.fields["general.description"] == "Simple addition"
    assert r.fields["general.name"] == "addition_op"
    assert [t.name for t in r.tensors] == ["x", "y", "result"]
    for t in r.tensors:
        assert t.tensor_type == 0 and t.dims == (3, 3) and t.n_elements == 9 and t.n_bytes == 36
    assert [t.data_offset for t in r.tensors] == [320, 384, 448]
    x, y, res = (r.tensor(n).data for n in ("x", "y", "result"))
    assert np.array_equal(res, x + y)
    assert abs(float(x[0, 0]) + float(y[0, 0]) - 0.070645) < 1e-6
    del x, y, res
    r.close()


def test_quantized_round_trip(tmp_path):
    path = str(tmp_path / "q.gguf")
    w4 = synth.weight(synth.Q4_K, 8, 512, seed=1)
    w6 = synth.weight(synth.Q6_K, 4, 256, seed=2)
    w8 = synth.weight(synth.Q8_0, 3, 96, seed=3)
    f = np.arange(6, dtype=np.float32).reshape(2, 3)
    h = np.arange(4, dtype=np.float16)
    gguf.write_gguf(path, {"general.architecture": "llama", "general.alignment": 64, "llama.rope.freq_base": 10000.0},
                    [("a.weight", 12, (8, 512), w4), ("b.weight", 14, (4, 256), w6), ("c.weight", 8, (3, 96), w8),
                     ("norm", 0, (2, 3), f), ("half", 1, (4,), h)], alignment=64)
    r = gguf.GGUFReader(path)
    assert r.alignment == 64 and r.data_offset % 64 == 0
    assert r.fields["llama.rope.freq_base"] == 10000.0
    a = r.tensor("a.weight")
    assert a.dims == (512, 8) and a.shape == (8, 512) and a.byte_shape == (8, 288) and a.n_bytes == 8 * 288
    assert np.array_equal(a.data, w4)
    assert np.array_equal(r.tensor("b.weight").data, w6) and r.tensor("b.weight").byte_shape == (4, 210)
    assert np.array_equal(r.tensor("c.weight").data, w8) and r.tensor("c.weight").byte_shape == (3, 102)
    assert np.array_equal(r.tensor("norm").data, f)
    assert np.array_equal(r.tensor("half").data, h)  # F16 is readable (the reference throws "No float16 in kotlin")
    # the bytes dequantize to the same values as the generator's
    assert np.array_equal(oracle_np.dequant(12, a.data), oracle_np.dequant(12, w4))
    assert all(t.data_offset % 64 == 0 for t in r.tensors)
    r.close()


def test_rejects_bad_files(tmp_path):
    p = tmp_path / "bad.gguf"
    p.write_bytes(b"GGUX" + b"\0" * 60)
    with pytest.raises(ValueError, match="GGUF magic invalid"):
        gguf.GGUFReader(str(p))
    p.write_bytes(struct.pack("<IIQQ", gguf.GGUF_MAGIC, 7, 0, 0))
    with pytest.raises(ValueError, match="Unsupported GGUF version: 7"):
        gguf.GGUFReader(str(p))
    gguf.write_gguf(str(p), {}, [("w", 12, (2, 256), synth.weight(12, 2, 256, seed=1)), ("w", 0, (1,), np.zeros(1, np.float32))])
    with pytest.raises(ValueError, match="Found duplicated tensor with name w"):
        gguf.GGUFReader(str(p))
    gguf.write_gguf(str(p), {}, [("w", 12, (2, 256), synth.weight(12, 2, 256, seed=1))])
    data = p.read_bytes()
    p.write_bytes(data[:-100])  # truncated data section
    with pytest.raises(ValueError, match="extends past the end"):
        gguf.GGUFReader(str(p))


def test_bad_row_size_message(tmp_path):
    p = str(tmp_path / "r.gguf")
    gguf.write_gguf(p, {}, [("w", 0, (2, 100), np.zeros((2, 100), np.float32))])
    r = gguf.GGUFReader(p)
    t = r.tensor("w")
    t.tensor_type = 12  # pretend: a Q4_K row of 100 elements
    with pytest.raises(ValueError, match=r"Quantized tensor row size \(100\) is not a multiple of Q4_K block size \(256\)"):
        _ = t.byte_shape
    del t
    r.close()
