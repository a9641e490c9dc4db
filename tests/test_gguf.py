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


def test_llama_config_and_weights_from_gguf(tmp_path):
    """A llama-architecture file written with the names and metadata keys of llama.cpp's files comes back as the
    decoder's configuration and weight table: grouped K / V heads, per-matrix types, shapes checked."""
    from skainet_amd import llama

    cfg = llama.Config(n_layer=2, hidden=512, ffn=768, n_head=4, n_kv_head=2, head_dim=128, vocab=256, max_tokens=64,
                       page_tokens=16, rope_base=50000.0, rms_eps=1e-6, type_embd=8,
                       matrix_types={"wv": 14, "l1.w_down": 8})
    w = llama.random_weights(cfg, seed=4)
    path = str(tmp_path / "tiny-llama.gguf")
    llama.write_gguf_model(path, cfg, w)
    r = gguf.GGUFReader(path)
    got = llama.config_from_gguf(r, page_tokens=16)
    for key in ("n_layer", "hidden", "ffn", "n_head", "n_kv_head", "head_dim", "vocab", "max_tokens", "rope_base"):
        assert getattr(got, key) == getattr(cfg, key), key
    assert abs(got.rms_eps - 1e-6) < 1e-12 and got.type_embd == 8
    gw = llama.weights_from_gguf(r, got)
    assert set(gw) == set(w)
    for name, (t, arr) in w.items():
        assert gw[name][0] == t, name
        assert np.array_equal(np.asarray(gw[name][1]).view(np.uint8).reshape(-1), np.asarray(arr).view(np.uint8).reshape(-1)), name
    assert gw["l0.wv"][0] == 14 and gw["l1.w_down"][0] == 8 and gw["l0.wk"][1].size == 2 * 128 * 2 * 144
    del gw
    r.close()
    # a file of another architecture, and one with a tensor of the wrong shape
    bad = str(tmp_path / "bad.gguf")
    gguf.write_gguf(bad, {"general.architecture": "gpt2"}, [("token_embd.weight", 0, (4, 4), np.zeros((4, 4), np.float32))])
    r = gguf.GGUFReader(bad)
    with pytest.raises(ValueError, match="only 'llama' files"):
        llama.config_from_gguf(r)
    r.close()

