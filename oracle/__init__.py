"""ctypes binding of the CPU oracle (``oracle/liboracle.so``).

TEST INFRASTRUCTURE: imported by tests, by ``__graft_entry__.smoke()`` and by
``bench.py``'s cpu_baseline leg only.  The product package never imports it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liboracle.so")

Q8_0, Q4_0, Q4_1, Q5_0, Q5_1, F16, F32, Q4_K, Q6_K, Q5_K = range(10)
TYPE_NAMES = {Q8_0: "Q8_0", Q4_0: "Q4_0", Q4_1: "Q4_1", Q5_0: "Q5_0", Q5_1: "Q5_1", F16: "F16", F32: "F32", Q4_K: "Q4_K", Q6_K: "Q6_K", Q5_K: "Q5_K"}


class ModelConfig(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("vocab_size", "hidden_size", "intermediate_size", "num_layers", "num_heads",
                                          "num_kv_heads", "head_dim", "max_seq_len")] + [("rms_norm_eps", C.c_float),
                                                                                         ("rope_theta", C.c_float),
                                                                                         ("sliding_window", C.c_int32)]


class SamplingConfig(C.Structure):
    _fields_ = [("temperature", C.c_float), ("top_k", C.c_int32), ("top_p", C.c_float), ("repetition_penalty", C.c_float),
                ("do_sample", C.c_int32)]


_lib = None


def build():
    subprocess.check_call(["make", "-C", _HERE, "-s", "liboracle.so"])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        vp, sz, i = C.c_void_p, C.c_size_t, C.c_int
        L.axo_f32_to_f16.restype, L.axo_f32_to_f16.argtypes = C.c_uint16, [C.c_float]
        L.axo_f16_to_f32.restype, L.axo_f16_to_f32.argtypes = C.c_float, [C.c_uint16]
        L.axo_f32_to_bf16.restype, L.axo_f32_to_bf16.argtypes = C.c_uint16, [C.c_float]
        L.axo_bf16_to_f32.restype, L.axo_bf16_to_f32.argtypes = C.c_float, [C.c_uint16]
        for f in ("axo_block_size", "axo_bytes_per_block"):
            getattr(L, f).restype, getattr(L, f).argtypes = sz, [i]
        for f in ("axo_num_blocks", "axo_packed_bytes"):
            getattr(L, f).restype, getattr(L, f).argtypes = sz, [i, sz]
        L.axo_quantize.restype, L.axo_quantize.argtypes = i, [i, vp, sz, vp]
        L.axo_dequantize.restype, L.axo_dequantize.argtypes = i, [i, vp, sz, vp]
        L.axo_matmul_ref.restype, L.axo_matmul_ref.argtypes = i, [i, vp, vp, vp, sz, sz, sz, vp, vp]
        L.axo_matmul_f64.restype, L.axo_matmul_f64.argtypes = None, [vp, vp, vp, sz, sz, sz, vp]
        L.axo_sgemm_wt.restype, L.axo_sgemm_wt.argtypes = None, [vp, vp, sz, sz, sz, vp]
        L.axo_num_threads.restype, L.axo_num_threads.argtypes = i, []
        L.axo_model_create.restype, L.axo_model_create.argtypes = vp, [C.POINTER(ModelConfig)]
        L.axo_model_free.restype, L.axo_model_free.argtypes = None, [vp]
        L.axo_model_set_embedding_f16.restype, L.axo_model_set_embedding_f16.argtypes = i, [vp, vp]
        L.axo_model_set_embedding_f32.restype, L.axo_model_set_embedding_f32.argtypes = i, [vp, vp]
        L.axo_model_set_norm.restype, L.axo_model_set_norm.argtypes = i, [vp, i, i, vp]
        L.axo_model_set_linear.restype, L.axo_model_set_linear.argtypes = i, [vp, i, i, i, vp]
        L.axo_model_forward.restype, L.axo_model_forward.argtypes = i, [vp, i, i, vp]
        L.axo_model_hidden.restype, L.axo_model_hidden.argtypes = C.POINTER(C.c_float), [vp]
        L.axo_model_kv.restype, L.axo_model_kv.argtypes = C.POINTER(C.c_uint16), [vp, i, i]
        L.axo_gguf_convert.restype, L.axo_gguf_convert.argtypes = i, [i, vp, vp, sz, sz, i]
        L.axo_ggml_dequantize.restype, L.axo_ggml_dequantize.argtypes = i, [i, vp, sz, vp]
        L.axo_get_next_token.restype, L.axo_get_next_token.argtypes = i, [vp, i, vp, i, C.POINTER(SamplingConfig), C.c_float]
        _lib = L
    return _lib


def packed_bytes(qtype, numel):
    return lib().axo_packed_bytes(qtype, numel)


def quantize(qtype, x):
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    out = np.zeros(packed_bytes(qtype, x.size), dtype=np.uint8)
    rc = lib().axo_quantize(qtype, x.ctypes.data, x.size, out.ctypes.data)
    if rc:
        raise ValueError(f"axo_quantize: {rc}")
    return out


def dequantize(qtype, packed, numel):
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    out = np.empty(numel, dtype=np.float32)
    rc = lib().axo_dequantize(qtype, packed.ctypes.data, numel, out.ctypes.data)
    if rc:
        raise ValueError(f"axo_dequantize: {rc}")
    return out


def matmul_ref(qtype, wq, x, n, k, bias=None):
    """The reference composition: dequantize -> transpose -> f32 sgemm (+bias)."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, k)
    m = x.shape[0]
    wq = np.ascontiguousarray(wq, dtype=np.uint8)
    y = np.empty((m, n), dtype=np.float32)
    scratch = np.empty(2 * n * k, dtype=np.float32)
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    rc = lib().axo_matmul_ref(qtype, wq.ctypes.data, x.ctypes.data, b.ctypes.data if b is not None else None, m, n, k,
                              y.ctypes.data, scratch.ctypes.data)
    if rc:
        raise ValueError(f"axo_matmul_ref: {rc}")
    return y


def matmul_f64(w_f32, x, bias=None):
    w = np.ascontiguousarray(w_f32, dtype=np.float32)
    n, k = w.shape
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, k)
    y = np.empty((x.shape[0], n), dtype=np.float64)
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    lib().axo_matmul_f64(w.ctypes.data, x.ctypes.data, b.ctypes.data if b is not None else None, x.shape[0], n, k,
                         y.ctypes.data)
    return y


def f32_to_f16_bits(x):
    L = lib()
    return np.array([L.axo_f32_to_f16(float(v)) for v in np.asarray(x, dtype=np.float32).reshape(-1)], dtype=np.uint16)


def f16_bits_to_f32(h):
    L = lib()
    return np.array([L.axo_f16_to_f32(int(v)) for v in np.asarray(h, dtype=np.uint16).reshape(-1)], dtype=np.float32)


class DecodeModel:
    """CPU decode oracle (oracle/axq_decode_oracle.c)."""

    LIN = {"q": 0, "k": 1, "v": 2, "o": 3, "gate": 4, "up": 5, "down": 6}

    def __init__(self, **cfg):
        self.cfg = ModelConfig(**cfg)
        self.h = lib().axo_model_create(C.byref(self.cfg))
        if not self.h:
            raise MemoryError("axo_model_create")

    def set_embedding_f16(self, table_bits):
        t = np.ascontiguousarray(table_bits, dtype=np.uint16)
        lib().axo_model_set_embedding_f16(self.h, t.ctypes.data)

    def set_embedding_f32(self, table):
        t = np.ascontiguousarray(table, dtype=np.float32)
        lib().axo_model_set_embedding_f32(self.h, t.ctypes.data)

    def set_norm(self, layer, which, w):
        w = np.ascontiguousarray(w, dtype=np.float32)
        lib().axo_model_set_norm(self.h, layer, which, w.ctypes.data)

    def set_linear(self, layer, which, qtype, packed):
        p = np.ascontiguousarray(packed, dtype=np.uint8)
        rc = lib().axo_model_set_linear(self.h, layer, which, qtype, p.ctypes.data)
        if rc:
            raise ValueError(f"axo_model_set_linear: {rc}")

    def forward(self, token, pos, want_logits=True):
        logits = np.empty(self.cfg.vocab_size, dtype=np.float32) if want_logits else None
        tok = lib().axo_model_forward(self.h, int(token), int(pos), logits.ctypes.data if want_logits else None)
        if tok < 0:
            raise ValueError("axo_model_forward: bad token or position")
        return tok, logits

    def hidden(self):
        return np.ctypeslib.as_array(lib().axo_model_hidden(self.h), shape=(self.cfg.hidden_size,)).copy()

    def kv(self, layer, which):
        c = self.cfg
        shape = (c.num_kv_heads, c.max_seq_len, c.head_dim)
        return np.ctypeslib.as_array(lib().axo_model_kv(self.h, layer, which), shape=shape).copy()

    def close(self):
        if self.h:
            lib().axo_model_free(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def gguf_convert(qtype, blocks, to_gguf):
    """Block images between ggml's order and the reference's (Q4_0 / Q4_1 permute nibbles, the rest copy)."""
    src = np.ascontiguousarray(blocks, dtype=np.uint8).reshape(-1)
    bb = lib().axo_bytes_per_block(qtype)
    assert src.size % bb == 0
    out = np.empty_like(src)
    rc = lib().axo_gguf_convert(qtype, src.ctypes.data, out.ctypes.data, src.size // bb, bb, 1 if to_gguf else 0)
    if rc:
        raise ValueError(f"axo_gguf_convert: {rc}")
    return out


def ggml_dequantize(qtype, blocks):
    """ggml's own row dequantiser on Q4_0 / Q4_1 blocks in ggml order."""
    src = np.ascontiguousarray(blocks, dtype=np.uint8).reshape(-1)
    nb = src.size // lib().axo_bytes_per_block(qtype)
    out = np.empty(nb * 32, dtype=np.float32)
    rc = lib().axo_ggml_dequantize(qtype, src.ctypes.data, nb, out.ctypes.data)
    if rc:
        raise ValueError(f"axo_ggml_dequantize: {rc}")
    return out


def get_next_token(logits, generated=(), temperature=1.0, top_k=None, top_p=None, repetition_penalty=1.0, do_sample=True, u=0.0):
    """TextGenerator::get_next_token with the uniform variate given; returns (token, filtered logits)."""
    work = np.array(logits, dtype=np.float32).reshape(-1)
    gen = np.ascontiguousarray(generated, dtype=np.int32).reshape(-1)
    cfg = SamplingConfig(temperature, top_k or 0, -1.0 if top_p is None else top_p, repetition_penalty, 1 if do_sample else 0)
    tok = lib().axo_get_next_token(work.ctypes.data, work.size, gen.ctypes.data if gen.size else None, gen.size, C.byref(cfg), u)
    return tok, work
