"""CPU: the built C-ABI library loads and exports every symbol that include/skainet_hip.h declares; the
host-only entry points (format table, status strings) behave like the reference's table; nothing here needs a GPU."""
import ctypes as C
import os
import re

import pytest

from skainet_amd import runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "skainet_hip.h")


def declared_symbols():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(skn_[a-z0-9_]+)\s*\(", src)))


def test_library_exports_every_declared_symbol():
    if not os.path.exists(runtime.LIB_PATH):
        pytest.fail(f"{runtime.LIB_PATH} has not been built (python -m skainet_amd.build)")
    lib = C.CDLL(runtime.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 40
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_binding_covers_the_header():
    assert sorted(runtime.exported_symbols()) == declared_symbols()
    runtime.load_library()  # resolves every bound symbol


def test_kotlin_ffm_binding_names_every_entry_point():
    """bindings/kotlin/jvm/SknLib.kt (source only: no JVM here) holds one downcall handle per declared function."""
    src = open(os.path.join(ROOT, "bindings", "kotlin", "jvm", "SknLib.kt")).read()
    assert sorted(re.findall(r'h\("(skn_[a-z0-9_]+)"', src)) == declared_symbols()
    for kt in ("jvm/QuantizedTensor.kt", "jvm/DeviceTensor.kt"):
        body = open(os.path.join(ROOT, "bindings", "kotlin", kt)).read()
        assert "TODO(" not in body
        # every member of the reference's Tensor interface (core/src/commonMain/kotlin/sk/ai/net/Tensor.kt:6-92)
        for member in ("plus(other: Tensor)", "plus(other: Double)", "plus(other: Int)", "minus(other: Double)",
                       "minus(other: Int)", "minus(other: Tensor)", "matmul(other: Tensor)", "fun t()", "fun relu()",
                       "softmax(dim: Int)", "fun softmax()", "pow(tensor: Tensor)", "pow(scalar: Double)", "fun sin()",
                       "fun cos()", "fun tan()", "fun asin()", "fun acos()", "fun atan()", "fun sinh()", "fun cosh()",
                       "fun tanh()", "fun exp()", "fun log()", "fun sqrt()", "fun cbrt()", "fun sigmoid()", "fun ln()",
                       "flatten(startDim: Int, endDim: Int)", "val shape", "val dataDescriptor"):
            assert member in body, (kt, member)


def test_format_table_matches_reference_constants():
    # reference gguf/src/commonMain/kotlin/sk/ai/net/gguf/Constants.kt:58-90 and Quants.kt:10-20
    assert runtime.type_block(runtime.Q8_0) == (32, 34)
    assert runtime.type_block(runtime.Q4_K) == (256, 144)
    assert runtime.type_block(runtime.Q6_K) == (256, 210)
    assert runtime.type_block(runtime.F32) == (1, 4)
    assert runtime.row_bytes(runtime.Q4_K, 11008) == 6192
    assert runtime.row_bytes(runtime.Q8_0, 4096) == 4352
    assert runtime.row_bytes(runtime.Q6_K, 4096) == 3360
    with pytest.raises(runtime.SknError) as e:
        runtime.row_bytes(runtime.Q4_K, 4100)
    assert e.value.code == runtime.ERR_SHAPE
    assert "row size (4100) is not a multiple of block size (256)" in e.value.message
    # every row of the reference's table: id -> (elements, bytes), Constants.kt:14-46 and :58-90
    qk = 256
    table = {
        0: (1, 4), 1: (1, 2), 2: (32, 2 + 16), 3: (32, 2 + 2 + 16), 6: (32, 2 + 4 + 16), 7: (32, 2 + 2 + 4 + 16),
        8: (32, 2 + 32), 9: (32, 4 + 4 + 32), 10: (256, 2 + 2 + qk // 16 + qk // 4), 11: (256, 2 + qk // 4 + qk // 8 + 12),
        12: (256, 2 + 2 + qk // 2 + 12), 13: (256, 2 + 2 + qk // 2 + qk // 8 + 12),
        14: (256, 2 + qk // 2 + qk // 4 + qk // 16), 15: (256, 4 + qk + qk // 8), 16: (256, 2 + qk // 4),
        17: (256, 2 + qk // 4 + qk // 32), 18: (256, 2 + qk // 4 + qk // 8), 19: (256, 2 + qk // 8 + qk // 16),
        20: (32, 2 + 16), 21: (256, 2 + qk // 4 + qk // 8 + qk // 32 + 4), 22: (256, 2 + qk // 4 + qk // 16),
        23: (256, 2 + 2 + qk // 2 + qk // 64), 24: (1, 1), 25: (1, 2), 26: (1, 4), 27: (1, 8), 28: (1, 8),
        29: (256, qk // 8 + qk // 16 + qk // 32), 30: (1, 2), 34: (256, 2 + 4 * 13), 35: (256, 2 + 64),
    }
    for type_id, sizes in table.items():
        assert runtime.type_block(type_id) == sizes, type_id
    for type_id in (4, 5, 31, 32, 33, 36, -1):  # ids the reference's enum does not have
        with pytest.raises(runtime.SknError) as e:
            runtime.type_block(type_id)
        assert e.value.code == runtime.ERR_TYPE


def test_status_strings_and_version():
    lib = runtime.load_library()
    assert lib.skn_abi_version() == 3
    assert lib.skn_status_string(0) == b"ok"
    assert lib.skn_status_string(-3) == b"shape mismatch"
    assert lib.skn_status_string(-99) == b"unknown status"


def test_no_device_fails_loudly_without_fallback():
    """Without a gfx950 device skn_init reports an error; no entry point computes on the CPU."""
    lib = runtime.load_library()
    h = C.c_void_p()
    rc = lib.skn_init(0, C.byref(h))
    if rc == 0:  # a GPU is present: nothing to check here
        lib.skn_shutdown(h)
        pytest.skip("a device is present")
    assert rc in (runtime.ERR_HIP, runtime.ERR_STATE)
    assert h.value is None
    assert lib.skn_last_error(None)
    # calls with a null context are rejected, never served by some host path
    assert lib.skn_dequant(None, 12, None, 256, None) == runtime.ERR_ARG
    assert lib.skn_matvec_q(None, 12, None, 1, 256, None, None) == runtime.ERR_ARG
