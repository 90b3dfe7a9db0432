"""ctypes binding of the axq C ABI (``include/axq.h``).

The shared library is built in-tree (``axonml_amd/libaxq.so``) by
``__graft_entry__.build()`` or ``make -C axonml_amd/csrc``.  There is no Python
or CPU fallback: if the library is missing, loading raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libaxq.so")

MEM_HOST, MEM_DEVICE = 0, 1


class AxqError(RuntimeError):
    """A non-zero axq_status, with the library's message."""

    def __init__(self, status, message):
        super().__init__(f"axq error {status}: {message}")
        self.status = status
        self.message = message


class DeviceInfo(C.Structure):
    _fields_ = [
        ("name", C.c_char * 128),
        ("arch", C.c_char * 32),
        ("compute_units", C.c_int32),
        ("wavefront_size", C.c_int32),
        ("lds_bytes_per_cu", C.c_int32),
        ("clock_mhz", C.c_int32),
        ("hbm_bytes", C.c_uint64),
    ]


class SamplingConfig(C.Structure):
    _fields_ = [("temperature", C.c_float), ("top_k", C.c_int32), ("top_p", C.c_float), ("repetition_penalty", C.c_float),
                ("do_sample", C.c_int32)]


class ModelConfig(C.Structure):
    _fields_ = [
        ("vocab_size", C.c_int32),
        ("hidden_size", C.c_int32),
        ("intermediate_size", C.c_int32),
        ("num_hidden_layers", C.c_int32),
        ("num_attention_heads", C.c_int32),
        ("num_key_value_heads", C.c_int32),
        ("head_dim", C.c_int32),
        ("max_position_embeddings", C.c_int32),
        ("rms_norm_eps", C.c_float),
        ("rope_theta", C.c_float),
        ("sliding_window", C.c_int32),
    ]


_vp, _sz, _i, _i64 = C.c_void_p, C.c_size_t, C.c_int, C.c_int64

# name -> (restype, argtypes): every symbol include/axq.h declares.
SIGNATURES = {
    "axq_type_block_size": (_sz, [_i]),
    "axq_type_bytes_per_block": (_sz, [_i]),
    "axq_type_bits_per_value": (_sz, [_i]),
    "axq_type_is_block_quantized": (_i, [_i]),
    "axq_type_name": (C.c_char_p, [_i]),
    "axq_type_from_str": (_i, [C.c_char_p]),
    "axq_num_blocks": (_sz, [_i, _sz]),
    "axq_packed_bytes": (_sz, [_i, _sz]),
    "axq_status_str": (C.c_char_p, [_i]),
    "axq_init": (_i, [_i, C.POINTER(_vp)]),
    "axq_destroy": (None, [_vp]),
    "axq_last_error": (C.c_char_p, [_vp]),
    "axq_device_info": (_i, [_vp, C.POINTER(DeviceInfo)]),
    "axq_malloc": (_i, [_vp, _sz, C.POINTER(_vp)]),
    "axq_free": (_i, [_vp, _vp]),
    "axq_copy_to_device": (_i, [_vp, _vp, _vp, _sz]),
    "axq_copy_to_host": (_i, [_vp, _vp, _vp, _sz]),
    "axq_copy_device_to_device": (_i, [_vp, _vp, _vp, _sz]),
    "axq_synchronize": (_i, [_vp]),
    "axq_set_stream": (_i, [_vp, _vp]),
    "axq_timer_start": (_i, [_vp]),
    "axq_timer_stop": (_i, [_vp, C.POINTER(C.c_float)]),
    "axq_quantize": (_i, [_vp, _i, _vp, _sz, _vp, _i]),
    "axq_dequantize": (_i, [_vp, _i, _vp, _sz, _vp, _i]),
    "axq_weight_upload": (_i, [_vp, _i, _i64, _i64, _vp, _sz, _i, C.POINTER(_vp)]),
    "axq_weight_quantize": (_i, [_vp, _i, _i64, _i64, _vp, _i, C.POINTER(_vp)]),
    "axq_weight_download": (_i, [_vp, _vp, _vp, _sz, _i]),
    "axq_weight_info": (_i, [_vp, C.POINTER(_i), C.POINTER(_i64), C.POINTER(_i64), C.POINTER(_sz)]),
    "axq_weight_free": (None, [_vp, _vp]),
    "axq_gemv_f32": (_i, [_vp, _vp, _vp, _i, _vp, _vp, _i]),
    "axq_gemv_f32_static": (_i, [_vp, _vp, _vp, _i, _vp, _vp]),
    "axq_gemm_bf16": (_i, [_vp, _vp, _vp, _i, _vp, _i]),
    "axq_model_create": (_i, [_vp, C.POINTER(ModelConfig), C.POINTER(_vp)]),
    "axq_model_free": (None, [_vp]),
    "axq_model_set_embedding_f16": (_i, [_vp, _vp, _i]),
    "axq_model_set_embedding_f32": (_i, [_vp, _vp, _i]),
    "axq_model_set_norm": (_i, [_vp, _i, _i, _vp, _i]),
    "axq_model_set_linear": (_i, [_vp, _i, _i, _vp]),
    "axq_model_random_init": (_i, [_vp, _i, C.c_float, C.c_uint64]),
    "axq_model_reset": (_i, [_vp]),
    "axq_model_forward": (_i, [_vp, C.c_int32, _vp, C.POINTER(C.c_int32)]),
    "axq_model_forward_tokens": (_i, [_vp, _vp, _i, _vp, C.POINTER(C.c_int32)]),
    "axq_model_generate": (_i, [_vp, _vp, _i, _i, _vp, C.POINTER(C.c_float), C.POINTER(C.c_float)]),
    "axq_model_seq_len": (_i, [_vp]),
    "axq_model_set_batch": (_i, [_vp, _i]),
    "axq_model_batch": (_i, [_vp]),
    "axq_model_copy_sequence": (_i, [_vp, _i, _i]),
    "axq_model_seq_len_of": (_i, [_vp, _i]),
    "axq_model_forward_batch": (_i, [_vp, _vp, _vp, _vp]),
    "axq_model_generate_batch": (_i, [_vp, _vp, _vp, _i, _vp, C.POINTER(C.c_float), C.POINTER(C.c_float)]),
    "axq_model_truncate": (_i, [_vp, _i]),
    "axq_model_read_hidden": (_i, [_vp, _vp]),
    "axq_model_read_kv": (_i, [_vp, _i, _i, _vp]),
    "axq_fill_normal_f32": (_i, [_vp, _vp, _sz, C.c_float, C.c_float, C.c_float, C.c_float, C.c_uint64]),
    "axq_bench_gemv_ring": (_i, [_vp, C.POINTER(_vp), _i, _i, _vp, _i, _vp, _i]),
    "axq_bench_read_ring": (_i, [_vp, C.POINTER(_vp), _i, _i, _vp, _i]),
    "axq_bench_read_ring_ex": (_i, [_vp, C.POINTER(_vp), _i, _i, _vp, _i, _i, _i, _i, _i, _i, _i]),
    "axq_bench_gemv_ring_streams": (_i, [_vp, C.POINTER(_vp), _i, _i, _vp, _i, _vp, _i, _i]),
    "axq_bench_graph_create": (_i, [_vp, C.POINTER(_vp), _i, _i, _vp, _i, _vp, _i, C.POINTER(_vp)]),
    "axq_bench_graph_create_read": (_i, [_vp, C.POINTER(_vp), _i, _i, _vp, _i, C.POINTER(_vp)]),
    "axq_bench_graph_launch": (_i, [_vp, _vp, _i]),
    "axq_bench_graph_destroy": (None, [_vp, _vp]),
    "axq_bench_copy": (_i, [_vp, _vp, _vp, _sz, _i]),
    "axq_bench_grid_barrier": (_i, [_vp, _i, _i, _i, C.POINTER(C.c_float)]),
    "axq_sample_token": (_i, [_vp, _vp, _i, _vp, _i, C.POINTER(SamplingConfig), C.c_float, C.POINTER(C.c_int32), _vp, _i]),
    "axq_model_set_sampling": (_i, [_vp, C.POINTER(SamplingConfig), C.c_uint64]),
    "axq_type_from_ggml": (_i, [_i]),
    "axq_type_to_ggml": (_i, [_i]),
    "axq_gguf_convert_blocks": (_i, [_vp, _i, _vp, _vp, _sz, _i, _i]),
}

_lib = None


def load_library():
    """Load libaxq.so (once) and attach the signatures.  Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `make -C axonml_amd/csrc` (hipcc, gfx950). There is no CPU fallback."
        )
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib
