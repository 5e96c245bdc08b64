"""ctypes binding of libcoeus_mi355x.so (the C ABI declared in include/coeus.h).

The library is the product: there is no Python or CPU fallback.  If the shared object is
missing or a call fails, an exception is raised.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libcoeus_mi355x.so")

OK, INVALID_INPUT, INVALID_CONFIG, DEVICE_ERROR, OUT_OF_MEMORY = range(5)
ACT_GELU_TANH, ACT_SILU_GATED = 0, 1
NORM_LAYERNORM, NORM_RMSNORM = 0, 1
SCOPE_SEQUENCE, SCOPE_TOKEN = 0, 1
W_F32, W_BF16, W_Q8_0, W_Q4_0 = 0, 1, 2, 3
KV_F32, KV_F16, KV_BF16 = 0, 1, 2
EPI_NONE, EPI_GELU, EPI_SILU_GATE = 0, 1, 2
MERGE_IN_KERNEL, MERGE_SEPARATE = 0, 1


class CSampling(C.Structure):
    _fields_ = [("temperature", C.c_float), ("top_k", C.c_uint32), ("top_p", C.c_float),
                ("seed", C.c_uint64)]


class CConfig(C.Structure):
    """coeus_config: Transformer250MConfig (CM:389-423) plus extension fields."""

    _fields_ = [
        ("hidden_dim", C.c_uint64), ("num_layers", C.c_uint64), ("num_heads", C.c_uint64),
        ("intermediate_dim", C.c_uint64), ("vocab_size", C.c_uint64),
        ("max_seq_len", C.c_uint64),
        ("dropout", C.c_float), ("attention_dropout", C.c_float),
        ("layer_norm_eps", C.c_float), ("use_bias", C.c_uint8),
        ("activation", C.c_uint32), ("norm", C.c_uint32), ("norm_scope", C.c_uint32),
        ("weight_dtype", C.c_uint32), ("kv_dtype", C.c_uint32),
        ("head_dim", C.c_uint64), ("max_batch", C.c_uint64),
    ]


# name -> (restype, argtypes); this table is also what the symbol-export test walks
_u64, _u32, _f32 = C.c_uint64, C.c_uint32, C.c_float
_vp, _cfgp = C.c_void_p, C.POINTER(CConfig)
SIGNATURES = {
    "coeus_last_error": (C.c_char_p, []),
    "coeus_device_info": (C.c_int, [C.c_char_p, _u64, C.POINTER(_u64), C.POINTER(_u32)]),
    "coeus_device_malloc": (C.c_int, [_u64, C.POINTER(_vp)]),
    "coeus_device_free": (C.c_int, [_vp]),
    "coeus_memcpy_h2d": (C.c_int, [_vp, _vp, _u64]),
    "coeus_memcpy_d2h": (C.c_int, [_vp, _vp, _u64]),
    "coeus_device_memset": (C.c_int, [_vp, C.c_int, _u64]),
    "coeus_device_copy": (C.c_int, [_vp, _vp, _u64, _vp]),
    "coeus_device_synchronize": (C.c_int, []),
    "coeus_stream_create": (C.c_int, [C.POINTER(_vp)]),
    "coeus_stream_synchronize": (C.c_int, [_vp]),
    "coeus_stream_destroy": (C.c_int, [_vp]),
    "coeus_event_create": (C.c_int, [C.POINTER(_vp)]),
    "coeus_event_record": (C.c_int, [_vp, _vp]),
    "coeus_event_synchronize": (C.c_int, [_vp]),
    "coeus_event_elapsed_ms": (C.c_int, [_vp, _vp, C.POINTER(_f32)]),
    "coeus_event_destroy": (C.c_int, [_vp]),
    "coeus_config_default": (None, [_cfgp]),
    "coeus_config_validate": (C.c_int, [_cfgp]),
    "coeus_config_num_parameters": (_u64, [_cfgp]),
    "coeus_config_used_parameters": (_u64, [_cfgp]),
    "coeus_init_default_parameters": (C.c_int, [_vp, _u64, _u64]),
    "coeus_positional_encoding": (C.c_int, [_u64, _u64, _vp]),
    "coeus_model_create": (C.c_int, [_cfgp, _vp, _u64, C.POINTER(_vp)]),
    "coeus_model_create_seeded": (C.c_int, [_cfgp, _u64, C.POINTER(_vp)]),
    "coeus_model_forward": (C.c_int, [_vp, _vp, _u64, _vp]),
    "coeus_model_forward_all": (C.c_int, [_vp, _vp, _u64, _vp]),
    "coeus_model_num_parameters": (_u64, [_vp]),
    "coeus_model_config": (_cfgp, [_vp]),
    "coeus_model_name": (C.c_char_p, [_vp]),
    "coeus_model_weight_bytes": (_u64, [_vp]),
    "coeus_model_resident_bytes": (_u64, [_vp]),
    "coeus_model_destroy": (None, [_vp]),
    "coeus_session_create": (C.c_int, [_vp, _u64, _u64, C.POINTER(_vp)]),
    "coeus_session_prefill": (C.c_int, [_vp, _vp, _u64, _vp]),
    "coeus_session_decode": (C.c_int, [_vp, _vp, _vp]),
    "coeus_session_decode_greedy": (C.c_int, [_vp, _vp, _u64, _vp]),
    "coeus_session_generate": (C.c_int, [_vp, _vp, _u64, _vp, _vp]),
    "coeus_op_sample": (C.c_int, [_vp, _u64, _u64, _vp, _u64, _vp, _vp]),
    "coeus_session_set_graph": (C.c_int, [_vp, C.c_int]),
    "coeus_session_graph_enabled": (C.c_int, [_vp]),
    "coeus_profiler_attached": (C.c_int, []),
    "coeus_session_time_decode_matmuls": (C.c_int, [_vp, _u64, C.POINTER(_f32), C.POINTER(_u64),
                                                    C.POINTER(_u64)]),
    "coeus_session_time_decode_attention": (C.c_int, [_vp, _u64, C.POINTER(_f32), C.POINTER(_u64),
                                                      C.POINTER(_u64)]),
    "coeus_session_position": (_u64, [_vp]),
    "coeus_session_reset": (C.c_int, [_vp]),
    "coeus_session_destroy": (None, [_vp]),
    "coeus_weight_create": (C.c_int, [_u32, _vp, _u64, _u64, C.POINTER(_vp)]),
    "coeus_weight_create_seeded": (C.c_int, [_u32, _u64, _u64, _u64, _u64, C.POINTER(_vp)]),
    "coeus_weight_dequantize": (C.c_int, [_vp, _vp]),
    "coeus_weight_bytes": (_u64, [_vp]),
    "coeus_weight_destroy": (None, [_vp]),
    "coeus_rustllm_checksum": (_u64, [_vp, _u64]),
    "coeus_rustllm_write": (C.c_int, [C.c_char_p, _vp, _vp, _u64]),
    "coeus_rustllm_read_header": (C.c_int, [C.c_char_p, _vp, C.POINTER(_u64)]),
    "coeus_rustllm_read_parameters": (C.c_int, [C.c_char_p, _vp, _u64]),
    "coeus_bpe_create": (C.c_int, [C.POINTER(_vp)]),
    "coeus_bpe_destroy": (None, [_vp]),
    "coeus_bpe_train": (C.c_int, [_vp, C.POINTER(C.c_char_p), C.POINTER(_u64), _u64, _u64]),
    "coeus_bpe_tokenize": (C.c_int, [_vp, C.c_char_p, _u64, _vp, _u64, C.POINTER(_u64), _vp, _u64, _vp,
                                     C.POINTER(_u64)]),
    "coeus_bpe_decode": (C.c_int, [C.c_char_p, _vp, _u64, _vp, _u64, C.POINTER(_u64)]),
    "coeus_bpe_vocab_size": (_u64, [_vp]),
    "coeus_bpe_num_merges": (_u64, [_vp]),
    "coeus_bpe_merge_rule": (C.c_int, [_vp, _u64, _vp, _u64, C.POINTER(_u64), _vp, _u64, C.POINTER(_u64)]),
    "coeus_bpe_add_token": (C.c_int, [_vp, C.c_char_p, _u64, C.POINTER(_u64)]),
    "coeus_bpe_remove_token": (C.c_int, [_vp, C.c_char_p, _u64]),
    "coeus_bpe_id_from_token": (C.c_int, [_vp, C.c_char_p, _u64, C.POINTER(_u64), C.POINTER(C.c_int)]),
    "coeus_bpe_token_from_id": (C.c_int, [_vp, _u64, _vp, _u64, C.POINTER(_u64), C.POINTER(C.c_int)]),
    "coeus_op_gemv": (C.c_int, [_vp, _vp, _u64, _vp, _vp, _u32, _vp, _vp]),
    "coeus_op_norm_gemv": (C.c_int, [_vp, _vp, _u64, _u32, _vp, _vp, _f32, _vp, _vp, _u32, _vp, C.POINTER(C.c_int),
                                     _vp]),
    "coeus_op_gemm": (C.c_int, [_vp, _vp, _u64, _vp, _vp, _u32, _vp, _vp]),
    "coeus_op_gemm_timed": (C.c_int, [_vp, _vp, _u64, _u32, _vp, _u32, _vp, _vp]),
    "coeus_op_norm": (C.c_int, [_u32, _u32, _vp, _u64, _u64, _vp, _vp, _f32, _vp, _vp]),
    "coeus_op_embed": (C.c_int, [_vp, _vp, _vp, _u64, _u64, _u64, _vp, _vp]),
    "coeus_op_attention": (C.c_int, [_vp, _u64, _u64, _u64, _vp, _vp]),
    "coeus_op_attention_decode": (C.c_int, [_vp, _vp, _vp, _u32, _u64, _u64, _u64, _u64, _u64, _u32, _u32, _vp,
                                            _vp]),
    "coeus_op_attention_decode_static": (C.c_int, [_vp, _vp, _vp, _u32, _u64, _u64, _u64, _u64, _u64, _u32, _u32,
                                                   _vp, _vp]),
}

_lib = None


def load():
    """Loads the shared library; raises if it has not been built."""
    global _lib
    if _lib is None:
        # COEUS_HOST_LIB names a build of the host-only sources (the sanitizer build): it exports
        # the entry points that never touch the device and nothing else
        host_only = os.environ.get("COEUS_HOST_LIB")
        path = host_only or LIB_PATH
        if not os.path.exists(path):
            raise ImportError(
                f"{path} is missing: build it with `python -m coeus_amd.build` "
                "(there is no CPU fallback)")
        lib = C.CDLL(path)
        for name, (res, args) in SIGNATURES.items():
            if host_only and not hasattr(lib, name):
                continue
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def last_error():
    return load().coeus_last_error().decode("utf-8", "replace")
