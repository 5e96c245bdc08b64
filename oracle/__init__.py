"""ctypes front-end of the CPU oracle (oracle/coeus_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg.  Nothing under coeus_amd/ imports this package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libcoeus_oracle.so")


def build(force=False):
    """Compile the oracle with gcc (no FMA contraction, no fast-math)."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


class Config(C.Structure):
    """Mirror of orc_config: Transformer250MConfig's fields (CM:389-423) + extensions."""

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


class Layout(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in (
        "token_embed_offset token_embed_size first_layer_offset layer_stride "
        "ln1_scale ln1_bias wq wk wv wo bq bk bv bo ln2_scale ln2_bias w_gate w_up w_down "
        "b_gate b_up b_down final_ln_offset output_proj_offset output_proj_size used_params "
        "total_params inner_dim").split()]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        f32p, u64p = C.POINTER(C.c_float), C.POINTER(C.c_uint64)
        cfgp = C.POINTER(Config)
        u64 = C.c_uint64
        sig = {
            "orc_set_threads": (None, [C.c_int]),
            "orc_config_default": (None, [cfgp]),
            "orc_config_validate": (C.c_int, [cfgp, C.POINTER(C.c_char_p)]),
            "orc_num_parameters": (u64, [cfgp]),
            "orc_param_layout": (None, [cfgp, C.POINTER(Layout)]),
            "orc_init_default": (None, [f32p, u64, u64]),
            "orc_matmul_ref": (None, [f32p, f32p, u64, u64, u64, f32p]),
            "orc_matmul": (None, [f32p, f32p, u64, u64, u64, f32p]),
            "orc_softmax": (None, [f32p, u64, f32p]),
            "orc_gelu": (C.c_float, [C.c_float]),
            "orc_layer_norm": (None, [f32p, u64, f32p, u64, f32p, u64, C.c_float, f32p]),
            "orc_positional_encoding": (None, [u64, u64, f32p]),
            "orc_causal_mask": (None, [u64, f32p]),
            "orc_mha_forward": (None, [u64, u64, f32p, f32p, f32p, f32p, f32p, f32p, u64, f32p]),
            "orc_ffn_forward": (None, [u64, u64, f32p, f32p, f32p, u64, f32p]),
            "orc_block_forward": (None, [u64, u64, u64] + [f32p] * 10 + [u64, C.c_float, f32p]),
            "orc_forward": (C.c_int, [cfgp, f32p, u64, u64p, u64, f32p, f32p, C.c_int]),
            "orc_bf16_round": (C.c_float, [C.c_float]),
            "orc_f32_to_f16": (C.c_uint16, [C.c_float]),
            "orc_f16_to_f32": (C.c_float, [C.c_uint16]),
            "orc_f16_round": (C.c_float, [C.c_float]),
            "orc_quantize_q8_0": (None, [f32p, u64, C.POINTER(C.c_int8), C.POINTER(C.c_uint16)]),
            "orc_dequantize_q8_0": (None, [C.POINTER(C.c_int8), C.POINTER(C.c_uint16), u64, f32p]),
            "orc_quantize_q4_0": (None, [f32p, u64, C.POINTER(C.c_uint8), C.POINTER(C.c_uint16)]),
            "orc_dequantize_q4_0": (None, [C.POINTER(C.c_uint8), C.POINTER(C.c_uint16), u64, f32p]),
            "orc_apply_weight_dtype": (None, [cfgp, f32p]),
            "orc_synth_normal": (C.c_float, [u64, u64]),
            "orc_init_seeded": (None, [cfgp, u64, f32p, u64]),
            "orc_synth_ids": (None, [u64, u64, u64p, u64]),
            "orc_session_create": (C.c_void_p, [cfgp, f32p, u64, u64]),
            "orc_session_destroy": (None, [C.c_void_p]),
            "orc_session_reset": (None, [C.c_void_p]),
            "orc_session_position": (u64, [C.c_void_p]),
            "orc_session_seek": (C.c_int, [C.c_void_p, u64]),
            "orc_session_set_literal_matmul": (None, [C.c_void_p, C.c_int]),
            "orc_session_feed": (C.c_int, [C.c_void_p, u64p, u64, f32p, f32p]),
            "orc_exp_nonpositive": (C.c_float, [C.c_float]),
            "orc_sample_u24": (C.c_uint32, [u64, u64, u64]),
            "orc_sample": (u64, [f32p, u64, C.c_uint32, C.c_float, C.c_float, u64, u64, u64]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def _f(a):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _u(a):
    return a.ctypes.data_as(C.POINTER(C.c_uint64))


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def set_threads(n):
    lib().orc_set_threads(int(n))


def default_config(**over):
    c = Config()
    lib().orc_config_default(C.byref(c))
    for k, v in over.items():
        setattr(c, k, v)
    return c


_ENUMS = dict(activation={"gelu": 0, "silu_gated": 1}, norm={"layernorm": 0, "rmsnorm": 1},
              norm_scope={"sequence": 0, "token": 1},
              weight_dtype={"f32": 0, "bf16": 1, "q8_0": 2, "q4_0": 3},
              kv_dtype={"f32": 0, "f16": 1, "bf16": 2})


def config_from_kwargs(kw):
    """Builds a Config from keyword values that may spell the enums as strings
    ("silu_gated", "rmsnorm", "token", "q4_0", "f16", ...)."""
    out = {}
    for k, v in kw.items():
        if k in _ENUMS and isinstance(v, str):
            v = _ENUMS[k][v]
        if k == "use_bias":
            v = 1 if v else 0
        out[k] = v
    return default_config(**out)


def validate(cfg):
    key = C.c_char_p()
    rc = lib().orc_config_validate(C.byref(cfg), C.byref(key))
    return rc, (key.value.decode() if key.value else None)


def num_parameters(cfg):
    return int(lib().orc_num_parameters(C.byref(cfg)))


def layout(cfg):
    L = Layout()
    lib().orc_param_layout(C.byref(cfg), C.byref(L))
    return L


def init_default(n, hidden_dim):
    p = np.empty(n, dtype=np.float32)
    lib().orc_init_default(_f(p), n, hidden_dim)
    return p


def init_seeded(cfg, seed, n=None):
    n = num_parameters(cfg) if n is None else n
    p = np.empty(n, dtype=np.float32)
    lib().orc_init_seeded(C.byref(cfg), seed, _f(p), n)
    return p


def synth_ids(seed, vocab, n):
    ids = np.empty(n, dtype=np.uint64)
    lib().orc_synth_ids(seed, vocab, _u(ids), n)
    return ids


def exp_nonpositive(x):
    return float(lib().orc_exp_nonpositive(float(x)))


def sample_u24(seed, position, row):
    return int(lib().orc_sample_u24(seed, position, row))


def sample(logits, top_k=0, top_p=0.0, temperature=1.0, seed=0, position=0, row=0):
    """The sampling specification (see coeus_oracle.h): one token id from one row of logits."""
    z = _f32(logits)
    return int(lib().orc_sample(_f(z), z.size, int(top_k), float(top_p), float(temperature), seed, position, row))


def matmul(a, b, ref=False):
    a, b = _f32(a), _f32(b)
    m, k = a.shape
    k2, n = b.shape
    assert k == k2
    c = np.empty((m, n), dtype=np.float32)
    (lib().orc_matmul_ref if ref else lib().orc_matmul)(_f(a), _f(b), m, n, k, _f(c))
    return c


def softmax(x):
    x = _f32(x)
    out = np.empty_like(x)
    lib().orc_softmax(_f(x), x.size, _f(out))
    return out


def gelu(x):
    return float(lib().orc_gelu(float(x)))


def layer_norm(x, scale, bias, eps):
    x, scale, bias = _f32(x), _f32(scale), _f32(bias)
    out = np.empty_like(x)
    lib().orc_layer_norm(_f(x), x.size, _f(scale), scale.size, _f(bias), bias.size, eps, _f(out))
    return out


def positional_encoding(max_seq_len, hidden_dim):
    t = np.empty((max_seq_len, hidden_dim), dtype=np.float32)
    lib().orc_positional_encoding(max_seq_len, hidden_dim, _f(t))
    return t


def causal_mask(s):
    m = np.empty((s, s), dtype=np.float32)
    lib().orc_causal_mask(s, _f(m))
    return m


def mha_forward(hidden, heads, q, k, v, weights, bias, mask, seq_len):
    q, k, v, weights = _f32(q), _f32(k), _f32(v), _f32(weights)
    bias = None if bias is None else _f32(bias)
    mask = None if mask is None else _f32(mask)
    out = np.empty(seq_len * hidden, dtype=np.float32)
    lib().orc_mha_forward(hidden, heads, _f(q), _f(k), _f(v), _f(weights),
                          _f(bias) if bias is not None else None,
                          _f(mask) if mask is not None else None, seq_len, _f(out))
    return out


def ffn_forward(hidden, inter, x, weights, bias, seq_len):
    x, weights = _f32(x), _f32(weights)
    bias = None if bias is None else _f32(bias)
    out = np.empty(seq_len * hidden, dtype=np.float32)
    lib().orc_ffn_forward(hidden, inter, _f(x), _f(weights),
                          _f(bias) if bias is not None else None, seq_len, _f(out))
    return out


def forward(cfg, params, ids, all_rows=False, fast=True, force_general=False):
    """Returns (rc, last_logits[, all_logits])."""
    params = _f32(params)
    ids = np.ascontiguousarray(ids, dtype=np.uint64)
    V = cfg.vocab_size
    last = np.zeros(V, dtype=np.float32)
    allr = np.zeros((len(ids), V), dtype=np.float32) if all_rows else None
    flags = (1 if fast else 0) | (2 if force_general else 0)
    rc = lib().orc_forward(C.byref(cfg), _f(params), params.size, _u(ids), len(ids), _f(last),
                           _f(allr) if all_rows else None, flags)
    return (rc, last, allr) if all_rows else (rc, last)


def bf16_round(x):
    x = _f32(x)
    u = x.view(np.uint32).astype(np.uint64)
    nan = ((u & 0x7F800000) == 0x7F800000) & ((u & 0x007FFFFF) != 0)
    r = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    r = np.where(nan, (u | 0x00400000) & 0xFFFF0000, r)
    return r.astype(np.uint32).view(np.float32).reshape(x.shape)


def quantize_q8_0(x):
    x = _f32(x).ravel()
    qs = np.empty(x.size, dtype=np.int8)
    ds = np.empty(x.size // 32, dtype=np.uint16)
    lib().orc_quantize_q8_0(_f(x), x.size, qs.ctypes.data_as(C.POINTER(C.c_int8)),
                            ds.ctypes.data_as(C.POINTER(C.c_uint16)))
    return qs, ds


def dequantize_q8_0(qs, ds):
    out = np.empty(qs.size, dtype=np.float32)
    lib().orc_dequantize_q8_0(qs.ctypes.data_as(C.POINTER(C.c_int8)),
                              ds.ctypes.data_as(C.POINTER(C.c_uint16)), qs.size, _f(out))
    return out


def quantize_q4_0(x):
    x = _f32(x).ravel()
    qs = np.empty(x.size // 2, dtype=np.uint8)
    ds = np.empty(x.size // 32, dtype=np.uint16)
    lib().orc_quantize_q4_0(_f(x), x.size, qs.ctypes.data_as(C.POINTER(C.c_uint8)),
                            ds.ctypes.data_as(C.POINTER(C.c_uint16)))
    return qs, ds


def dequantize_q4_0(qs, ds):
    out = np.empty(qs.size * 2, dtype=np.float32)
    lib().orc_dequantize_q4_0(qs.ctypes.data_as(C.POINTER(C.c_uint8)),
                              ds.ctypes.data_as(C.POINTER(C.c_uint16)), qs.size * 2, _f(out))
    return out


def apply_weight_dtype(cfg, params):
    """Returns a copy of params with linear weights round-tripped through cfg.weight_dtype."""
    p = _f32(params).copy()
    lib().orc_apply_weight_dtype(C.byref(cfg), _f(p))
    return p


class Session:
    """KV-cache incremental forward (per-token norm scope only)."""

    def __init__(self, cfg, params, max_ctx):
        self.cfg = cfg
        self.params = _f32(params)  # keep alive: the C side borrows the pointer
        self.h = lib().orc_session_create(C.byref(cfg), _f(self.params), self.params.size, max_ctx)
        if not self.h:
            raise ValueError("orc_session_create failed (norm_scope must be 1, sizes in range)")

    def feed(self, ids, all_rows=False):
        ids = np.ascontiguousarray(ids, dtype=np.uint64)
        V = self.cfg.vocab_size
        last = np.zeros(V, dtype=np.float32)
        allr = np.zeros((len(ids), V), dtype=np.float32) if all_rows else None
        rc = lib().orc_session_feed(self.h, _u(ids), len(ids), _f(last),
                                    _f(allr) if all_rows else None)
        return (rc, last, allr) if all_rows else (rc, last)

    @property
    def position(self):
        return int(lib().orc_session_position(self.h))

    def reset(self):
        lib().orc_session_reset(self.h)

    def seek(self, pos):
        return lib().orc_session_seek(self.h, pos)

    def set_literal_matmul(self, on):
        lib().orc_session_set_literal_matmul(self.h, 1 if on else 0)

    def close(self):
        if self.h:
            lib().orc_session_destroy(self.h)
            self.h = None

    def __del__(self):
        self.close()
