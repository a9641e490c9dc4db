"""ctypes binding of libskainet_hip.so -- the same C ABI a Kotlin cinterop / Panama FFM binding would use.

There is no CPU fallback: if the library is missing or no gfx950 device is present the calls raise.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libskainet_hip.so")

F32, F16, Q8_0, Q4_K, Q6_K = 0, 1, 8, 12, 14
Q4_0, Q4_1, Q5_0, Q5_1, Q2_K, Q5_K, BF16 = 2, 3, 6, 7, 10, 13, 30
Q3_K, Q8_K, IQ4_NL, IQ4_XS = 11, 15, 20, 23
TQ1_0, TQ2_0 = 34, 35

OK = 0
ERR_ARG, ERR_TYPE, ERR_SHAPE, ERR_OOM, ERR_HIP, ERR_RANGE, ERR_POOL, ERR_STATE = -1, -2, -3, -4, -5, -6, -7, -8


class SknError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"[{code}] {message}")
        self.code = code
        self.message = message


class LlamaConfig(C.Structure):
    _fields_ = [
        ("n_layer", C.c_int32), ("hidden", C.c_int32), ("ffn", C.c_int32), ("n_head", C.c_int32),
        ("head_dim", C.c_int32), ("vocab", C.c_int32), ("max_tokens", C.c_int32), ("page_tokens", C.c_int32),
        ("rope_base", C.c_float), ("rms_eps", C.c_float), ("n_kv_head", C.c_int32),
    ]


class LlamaLayer(C.Structure):
    _fields_ = [
        ("wq", C.c_void_p), ("wo", C.c_void_p), ("wk", C.c_void_p), ("wv", C.c_void_p),
        ("w_gate", C.c_void_p), ("w_up", C.c_void_p), ("w_down", C.c_void_p),
        ("attn_norm", C.c_void_p), ("ffn_norm", C.c_void_p),
        ("type_q", C.c_int32), ("type_k", C.c_int32), ("type_v", C.c_int32), ("type_o", C.c_int32),
        ("type_gate", C.c_int32), ("type_up", C.c_int32), ("type_down", C.c_int32),
    ]


class LlamaWeights(C.Structure):
    _fields_ = [
        ("tok_embd", C.c_void_p), ("out_norm", C.c_void_p), ("out_head", C.c_void_p),
        ("type_embd", C.c_int32), ("type_head", C.c_int32),
        ("layers", C.POINTER(LlamaLayer)),
    ]


_SIGNATURES = {
    # name: (restype, argtypes)
    "skn_synth_weight": (C.c_int, [C.c_int, C.c_int64, C.c_int64, C.c_uint64, C.c_void_p, C.c_size_t]),
    "skn_synth_activation_f32": (C.c_int, [C.c_int64, C.c_uint64, C.c_void_p]),
    "skn_synth_activation_bf16": (C.c_int, [C.c_int64, C.c_uint64, C.c_void_p]),
    "skn_synth_kv_f16": (C.c_int, [C.c_int64, C.c_uint64, C.c_void_p]),
    "skn_synth_checksum": (C.c_uint64, [C.c_void_p, C.c_size_t]),
    "skn_abi_version": (C.c_int, []),
    "skn_init": (C.c_int, [C.c_int, C.POINTER(C.c_void_p)]),
    "skn_shutdown": (None, [C.c_void_p]),
    "skn_last_error": (C.c_char_p, [C.c_void_p]),
    "skn_status_string": (C.c_char_p, [C.c_int]),
    "skn_device_info": (C.c_int, [C.c_void_p, C.c_char_p, C.c_size_t, C.POINTER(C.c_int), C.POINTER(C.c_size_t)]),
    "skn_type_block": (C.c_int, [C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "skn_row_bytes": (C.c_int64, [C.c_int, C.c_int64]),
    "skn_malloc": (C.c_int, [C.c_void_p, C.c_size_t, C.POINTER(C.c_void_p)]),
    "skn_free": (C.c_int, [C.c_void_p, C.c_void_p]),
    "skn_upload": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]),
    "skn_download": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]),
    "skn_memset": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_size_t]),
    "skn_copy": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]),
    "skn_sync": (C.c_int, [C.c_void_p]),
    "skn_set_stream": (C.c_int, [C.c_void_p, C.c_void_p]),
    "skn_set_option": (C.c_int, [C.c_void_p, C.c_char_p, C.c_int]),
    "skn_test_fused_matvec": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_int,
                                        C.c_int, C.c_void_p, C.c_void_p, C.c_float, C.c_void_p, C.c_void_p, C.c_void_p, C.c_float]),
    "skn_get_stat": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(C.c_int64)]),
    "skn_timer_start": (C.c_int, [C.c_void_p]),
    "skn_timer_stop": (C.c_int, [C.c_void_p, C.POINTER(C.c_float)]),
    "skn_prof_start": (C.c_int, [C.c_void_p, C.c_int]),
    "skn_prof_stop": (C.c_int, [C.c_void_p, C.POINTER(C.c_double), C.POINTER(C.c_int)]),
    "skn_dequant": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p, C.c_int64, C.c_void_p]),
    "skn_matvec_q": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p]),
    "skn_gemm_q": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_void_p]),
    "skn_gemm_expanded_bytes": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_size_t)]),
    "skn_gemm_expand": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p]),
    "skn_gemm_expanded": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_void_p]),
    "skn_test_matvec_q4k_stamps": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]),
    "skn_kv_create": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_void_p)]),
    "skn_kv_free": (C.c_int, [C.c_void_p, C.c_void_p]),
    "skn_kv_reset": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int]),
    "skn_kv_len": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int]),
    "skn_kv_append": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(C.c_int32), C.c_int]),
    "skn_kv_append_run": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int]),
    "skn_kv_gather": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]),
    "skn_attn_decode": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(C.c_int32), C.c_float, C.c_void_p]),
    "skn_attn_decode_static": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_float, C.c_void_p]),
    "skn_attn_prefill": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_float, C.c_void_p]),
    "skn_rmsnorm": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_float, C.c_void_p]),
    "skn_rope": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float]),
    "skn_swiglu": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]),
    "skn_relu": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]),
    "skn_add_inplace": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64]),
    "skn_argmax": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p]),
    "skn_f32_to_f16": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]),
    "skn_f32_to_bf16": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]),
    "skn_llama_create": (C.c_int, [C.c_void_p, C.POINTER(LlamaConfig), C.POINTER(LlamaWeights), C.POINTER(C.c_void_p)]),
    "skn_llama_free": (C.c_int, [C.c_void_p, C.c_void_p]),
    "skn_llama_reset": (C.c_int, [C.c_void_p, C.c_void_p]),
    "skn_llama_prefill": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(C.c_int32), C.c_int, C.POINTER(C.c_int32)]),
    "skn_llama_decode": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int, C.POINTER(C.c_int32)]),
    "skn_llama_logits": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(C.c_void_p)]),
}

_LIB = None


def load_library():
    """Loads the in-tree library; raises with the build command when it has not been built."""
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m skainet_amd.build` (needs hipcc); "
                "there is no CPU fallback for the HIP path"
            )
        lib = C.CDLL(LIB_PATH)
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _LIB = lib
    return _LIB


def exported_symbols():
    return list(_SIGNATURES)


def type_block(ggml_type):
    be, bb = C.c_int(), C.c_int()
    lib = load_library()
    rc = lib.skn_type_block(ggml_type, C.byref(be), C.byref(bb))
    if rc != OK:
        raise SknError(rc, lib.skn_last_error(None).decode())
    return be.value, bb.value


def row_bytes(ggml_type, k):
    lib = load_library()
    rc = lib.skn_row_bytes(ggml_type, k)
    if rc < 0:
        raise SknError(int(rc), lib.skn_last_error(None).decode())
    return int(rc)


def synth_weight(ggml_type, n_rows, k, seed):
    """skn_synth_weight: the library's seeded blocks of an [n_rows, k] weight (host array; needs no device)."""
    lib = load_library()
    out = np.empty(n_rows * row_bytes(ggml_type, k), dtype=np.uint8)
    rc = lib.skn_synth_weight(ggml_type, n_rows, k, seed, out.ctypes.data, out.nbytes)
    if rc != OK:
        raise SknError(rc, lib.skn_last_error(None).decode())
    return out


def _synth_vector(name, dtype, n, seed):
    lib = load_library()
    out = np.empty(n, dtype=dtype)
    rc = getattr(lib, name)(n, seed, out.ctypes.data)
    if rc != OK:
        raise SknError(rc, lib.skn_last_error(None).decode())
    return out


def synth_activation_f32(n, seed):
    return _synth_vector("skn_synth_activation_f32", np.float32, n, seed)


def synth_activation_bf16(n, seed):
    return _synth_vector("skn_synth_activation_bf16", np.uint16, n, seed)


def synth_kv_f16(n, seed):
    return _synth_vector("skn_synth_kv_f16", np.uint16, n, seed)


def synth_checksum(arr):
    a = np.ascontiguousarray(arr)
    return int(load_library().skn_synth_checksum(a.ctypes.data, a.nbytes))


class DeviceBuffer:
    """Owned device allocation.  `ptr` is the raw device address (an int)."""

    def __init__(self, ctx, nbytes):
        self.ctx = ctx
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        ctx._check(ctx.lib.skn_malloc(ctx.handle, self.nbytes, C.byref(p)))
        self.ptr = p.value or 0

    def upload(self, array, offset=0):
        a = np.ascontiguousarray(array)
        if offset + a.nbytes > self.nbytes:
            raise ValueError("upload exceeds the buffer")
        self.ctx._check(self.ctx.lib.skn_upload(self.ctx.handle, self.ptr + offset, a.ctypes.data, a.nbytes))
        return self

    def download(self, dtype, count=None, offset=0):
        dt = np.dtype(dtype)
        if count is None:
            count = (self.nbytes - offset) // dt.itemsize
        out = np.empty(count, dtype=dt)
        if out.nbytes + offset > self.nbytes:
            raise ValueError("download exceeds the buffer")
        self.ctx._check(self.ctx.lib.skn_download(self.ctx.handle, out.ctypes.data, self.ptr + offset, out.nbytes))
        return out

    def free(self):
        if self.ptr:
            self.ctx.lib.skn_free(self.ctx.handle, self.ptr)
            self.ptr = 0

    def __del__(self):
        try:
            if self.ptr and self.ctx.handle:
                self.free()
        except Exception:
            pass


class KVCache:
    def __init__(self, ctx, n_seq, n_head, head_dim, page_tokens, max_tokens):
        self.ctx = ctx
        self.n_seq, self.n_head, self.head_dim = n_seq, n_head, head_dim
        self.page_tokens, self.max_tokens = page_tokens, max_tokens
        h = C.c_void_p()
        ctx._check(ctx.lib.skn_kv_create(ctx.handle, n_seq, n_head, head_dim, page_tokens, max_tokens, C.byref(h)))
        self.handle = h.value

    def length(self, seq):
        rc = self.ctx.lib.skn_kv_len(self.ctx.handle, self.handle, seq)
        if rc < 0:
            self.ctx._check(rc)
        return rc

    def reset(self, seq=-1):
        self.ctx._check(self.ctx.lib.skn_kv_reset(self.ctx.handle, self.handle, seq))

    def append(self, k_dev, v_dev, seq_ids):
        ids = (C.c_int32 * len(seq_ids))(*seq_ids)
        self.ctx._check(self.ctx.lib.skn_kv_append(self.ctx.handle, self.handle, _ptr(k_dev), _ptr(v_dev), ids, len(seq_ids)))

    def append_run(self, seq, k_dev, v_dev, n_tokens):
        self.ctx._check(self.ctx.lib.skn_kv_append_run(self.ctx.handle, self.handle, seq, _ptr(k_dev), _ptr(v_dev), n_tokens))

    def gather(self, seq, t0, t1, k_out_dev, v_out_dev):
        self.ctx._check(self.ctx.lib.skn_kv_gather(self.ctx.handle, self.handle, seq, t0, t1, _ptr(k_out_dev), _ptr(v_out_dev)))

    def attn_decode(self, q_dev, out_dev, scale, n_ctx=None):
        arr = None if n_ctx is None else (C.c_int32 * len(n_ctx))(*[int(v) for v in n_ctx])
        if n_ctx is not None and len(n_ctx) != self.n_seq:
            raise ValueError("n_ctx needs one entry per sequence")
        self.ctx._check(self.ctx.lib.skn_attn_decode(self.ctx.handle, self.handle, _ptr(q_dev), arr, scale, _ptr(out_dev)))

    def attn_decode_static(self, q_dev, out_dev, scale):
        """skn_attn_decode over all cached tokens with the library's static scratch (allocates nothing)."""
        self.ctx._check(self.ctx.lib.skn_attn_decode_static(self.ctx.handle, self.handle, _ptr(q_dev), scale, _ptr(out_dev)))

    def attn_prefill(self, seq, q_dev, n_queries, out_dev, scale):
        """Causal attention of the last n_queries tokens of sequence seq (q/out fp32 [n_queries][n_head][head_dim])."""
        self.ctx._check(self.ctx.lib.skn_attn_prefill(self.ctx.handle, self.handle, int(seq), _ptr(q_dev), int(n_queries),
                                                      scale, _ptr(out_dev)))

    def free(self):
        if self.handle:
            self.ctx.lib.skn_kv_free(self.ctx.handle, self.handle)
            self.handle = None

    def __del__(self):
        try:
            if self.handle and self.ctx.handle:
                self.free()
        except Exception:
            pass


def _ptr(x):
    if isinstance(x, DeviceBuffer):
        return x.ptr
    if x is None:
        return None
    return int(x)


class Context:
    """One skn_ctx: a device, a stream, and the error slot."""

    def __init__(self, device=0):
        self.lib = load_library()
        h = C.c_void_p()
        rc = self.lib.skn_init(device, C.byref(h))
        if rc != OK:
            raise SknError(rc, self.lib.skn_last_error(None).decode())
        self.handle = h.value

    def _check(self, rc):
        if rc != OK:
            raise SknError(rc, self.lib.skn_last_error(self.handle).decode())

    def close(self):
        if self.handle:
            self.lib.skn_shutdown(self.handle)
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    # -- memory ---------------------------------------------------------------------------------
    def alloc(self, nbytes):
        return DeviceBuffer(self, nbytes)

    def to_device(self, array):
        a = np.ascontiguousarray(array)
        return DeviceBuffer(self, max(a.nbytes, 16)).upload(a)

    def sync(self):
        self._check(self.lib.skn_sync(self.handle))

    def memset(self, dev, byte_value, nbytes):
        self._check(self.lib.skn_memset(self.handle, _ptr(dev), int(byte_value), nbytes))

    def copy(self, dst_dev, src_dev, nbytes):
        self._check(self.lib.skn_copy(self.handle, _ptr(dst_dev), _ptr(src_dev), nbytes))

    def set_stream(self, stream_ptr):
        self._check(self.lib.skn_set_stream(self.handle, stream_ptr))

    def device_info(self):
        name = C.create_string_buffer(256)
        cus, total = C.c_int(), C.c_size_t()
        self._check(self.lib.skn_device_info(self.handle, name, 256, C.byref(cus), C.byref(total)))
        return {"name": name.value.decode(), "compute_units": cus.value, "total_bytes": total.value}

    def timer_start(self):
        self._check(self.lib.skn_timer_start(self.handle))

    def timer_stop(self):
        ms = C.c_float()
        self._check(self.lib.skn_timer_stop(self.handle, C.byref(ms)))
        return ms.value

    def set_option(self, key, value):
        self._check(self.lib.skn_set_option(self.handle, key.encode(), int(value)))

    def test_fused_matvec(self, ggml_type, epi, mats, k, x_dev, norm_w_dev, eps, y_dev, kv=None, pos_dev=None, rope_base=10000.0):
        """mats: up to three (device buffer, rows) pairs."""
        mats = list(mats) + [(None, 0)] * (3 - len(mats))
        args = []
        for buf, rows in mats:
            args += [_ptr(buf), int(rows)]
        self._check(self.lib.skn_test_fused_matvec(self.handle, ggml_type, epi, *args, k, _ptr(x_dev), _ptr(norm_w_dev), eps,
                                                   _ptr(y_dev), kv.handle if kv is not None else None, _ptr(pos_dev), rope_base))

    def stat(self, key):
        v = C.c_int64()
        self._check(self.lib.skn_get_stat(self.handle, key.encode(), C.byref(v)))
        return v.value

    def prof_start(self, max_launches):
        self._check(self.lib.skn_prof_start(self.handle, max_launches))

    def prof_stop(self):
        """-> (summed kernel milliseconds, launches timed)"""
        ms, n = C.c_double(), C.c_int()
        self._check(self.lib.skn_prof_stop(self.handle, C.byref(ms), C.byref(n)))
        return ms.value, n.value

    # -- ops on device pointers --------------------------------------------------------------------
    def dequant(self, ggml_type, w_dev, n_elems, out_dev):
        self._check(self.lib.skn_dequant(self.handle, ggml_type, _ptr(w_dev), n_elems, _ptr(out_dev)))

    def matvec_q(self, ggml_type, w_dev, n, k, x_dev, y_dev):
        self._check(self.lib.skn_matvec_q(self.handle, ggml_type, _ptr(w_dev), n, k, _ptr(x_dev), _ptr(y_dev)))

    def gemm_q(self, ggml_type, w_dev, n, k, a_bf16_dev, m, c_dev):
        self._check(self.lib.skn_gemm_q(self.handle, ggml_type, _ptr(w_dev), n, k, _ptr(a_bf16_dev), m, _ptr(c_dev)))

    def gemm_expanded_bytes(self, ggml_type, n, k):
        out = C.c_size_t(0)
        self._check(self.lib.skn_gemm_expanded_bytes(self.handle, ggml_type, n, k, C.byref(out)))
        return int(out.value)

    def gemm_expand(self, ggml_type, w_dev, n, k):
        """-> device buffer with the expanded copy of W [n, k] that gemm_expanded multiplies with."""
        buf = self.alloc(max(self.gemm_expanded_bytes(ggml_type, n, k), 16))
        self._check(self.lib.skn_gemm_expand(self.handle, ggml_type, _ptr(w_dev), n, k, _ptr(buf)))
        return buf

    def gemm_expanded(self, expanded_dev, n, k, a_bf16_dev, m, c_dev):
        self._check(self.lib.skn_gemm_expanded(self.handle, _ptr(expanded_dev), n, k, _ptr(a_bf16_dev), m, _ptr(c_dev)))

    def test_matvec_q4k_stamps(self, w_dev, n, k, x_dev, y_dev, stamps_dev):
        """The Q4_K matvec with the kernel's measuring build: eight 64-bit stamps per row in stamps_dev."""
        self._check(self.lib.skn_test_matvec_q4k_stamps(self.handle, _ptr(w_dev), n, k, _ptr(x_dev), _ptr(y_dev), _ptr(stamps_dev)))

    def rmsnorm(self, x_dev, w_dev, rows, n, eps, y_dev):
        self._check(self.lib.skn_rmsnorm(self.handle, _ptr(x_dev), _ptr(w_dev), rows, n, eps, _ptr(y_dev)))

    def rope(self, x_dev, rows, n_head, head_dim, pos0, base):
        self._check(self.lib.skn_rope(self.handle, _ptr(x_dev), rows, n_head, head_dim, pos0, base))

    def swiglu(self, gate_dev, up_dev, n, out_dev):
        self._check(self.lib.skn_swiglu(self.handle, _ptr(gate_dev), _ptr(up_dev), n, _ptr(out_dev)))

    def relu(self, x_dev, n, out_dev):
        self._check(self.lib.skn_relu(self.handle, _ptr(x_dev), n, _ptr(out_dev)))

    def add_inplace(self, y_dev, x_dev, n):
        self._check(self.lib.skn_add_inplace(self.handle, _ptr(y_dev), _ptr(x_dev), n))

    def argmax(self, x_dev, n, index_dev):
        self._check(self.lib.skn_argmax(self.handle, _ptr(x_dev), n, _ptr(index_dev)))

    def f32_to_f16(self, x_dev, n, out_dev):
        self._check(self.lib.skn_f32_to_f16(self.handle, _ptr(x_dev), n, _ptr(out_dev)))

    def f32_to_bf16(self, x_dev, n, out_dev):
        self._check(self.lib.skn_f32_to_bf16(self.handle, _ptr(x_dev), n, _ptr(out_dev)))

    def kv_cache(self, n_seq, n_head, head_dim, page_tokens, max_tokens):
        return KVCache(self, n_seq, n_head, head_dim, page_tokens, max_tokens)

    # -- host-array conveniences (upload, run, download) used by tests and the smoke check ---------
    def dequant_host(self, ggml_type, raw):
        raw = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
        be, bb = type_block(ggml_type)
        if raw.size % bb:
            raise SknError(ERR_SHAPE, "byte count is not a whole number of blocks")
        n = raw.size // bb * be
        w = self.to_device(raw)
        out = self.alloc(max(4 * n, 16))
        self.dequant(ggml_type, w, n, out)
        return out.download(np.float32, n)

    def matvec_q_host(self, ggml_type, raw, n, k, x):
        w = self.to_device(np.ascontiguousarray(raw).view(np.uint8))
        xd = self.to_device(np.ascontiguousarray(x, dtype=np.float32))
        yd = self.alloc(max(4 * n, 16))
        self.matvec_q(ggml_type, w, n, k, xd, yd)
        return yd.download(np.float32, n)

    def gemm_q_host(self, ggml_type, raw, n, k, a_bf16, m):
        w = self.to_device(np.ascontiguousarray(raw).view(np.uint8))
        ad = self.to_device(np.ascontiguousarray(a_bf16, dtype=np.uint16))
        cd = self.alloc(max(4 * n * m, 16))
        self.gemm_q(ggml_type, w, n, k, ad, m, cd)
        return cd.download(np.float32, n * m).reshape(m, n)
