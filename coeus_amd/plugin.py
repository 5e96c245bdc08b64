"""Host-side mirror of the reference's plugin surface for the transformer forward path:

    TransformerModelPlugin().create_builder().build(config) -> model;  model.forward(token_ids)

(rustllm-core/plugins/model-transformer/src/lib.rs:503-533, 583-638, 787-924), implemented
over the C ABI of libcoeus_mi355x.so.  Names, argument meaning and error behaviour follow the
reference; `Result<T>` becomes "return T or raise".  All arithmetic runs on the GPU.
"""
import ctypes as C
from dataclasses import dataclass, fields

import numpy as np

from . import _lib
from ._lib import CConfig


# ---------------------------------------------------------------- errors
class CoeusError(Exception):
    """rustllm_core::foundation::error::Error (foundation/error.rs:17-44)."""


class ProcessingError(CoeusError):
    """Error::Processing(ProcessingError::InvalidInput { description, position: None })."""


class ConfigError(CoeusError):
    """Error::Config(ConfigError::Invalid { key, value, error })."""


class DeviceError(CoeusError):
    """internal_error(..) (foundation/error.rs:650-655): the device or an allocation failed."""


def _check(rc):
    if rc == _lib.OK:
        return
    msg = _lib.last_error()
    if rc == _lib.INVALID_INPUT:
        raise ProcessingError(msg)
    if rc == _lib.INVALID_CONFIG:
        raise ConfigError(msg)
    raise DeviceError(msg)


# ---------------------------------------------------------------- config
@dataclass
class Transformer250MConfig:
    """Transformer250MConfig (core/model.rs:389-423) with its Default (core/model.rs:534-550).

    The trailing fields are extensions; their defaults reproduce the reference."""

    hidden_dim: int = 768
    num_layers: int = 12
    num_heads: int = 12
    intermediate_dim: int = 3072
    vocab_size: int = 50257
    max_seq_len: int = 1024
    dropout: float = 0.1
    attention_dropout: float = 0.1
    layer_norm_eps: float = 1e-5
    use_bias: bool = True
    activation: str = "gelu"          # "gelu" | "silu_gated" (the reference ignores the string)
    # extensions
    norm: str = "layernorm"           # "layernorm" | "rmsnorm"
    norm_scope: str = "sequence"      # "sequence" (reference, lib.rs:105-128) | "token"
    weight_dtype: str = "f32"         # "f32" | "bf16" | "q8_0" | "q4_0"
    kv_dtype: str = "f32"             # "f32" | "f16" | "bf16"
    head_dim: int = 0                 # 0 => hidden_dim // num_heads
    max_batch: int = 1

    _ACT = {"gelu": 0, "silu_gated": 1}
    _NORM = {"layernorm": 0, "rmsnorm": 1}
    _SCOPE = {"sequence": 0, "token": 1}
    _WD = {"f32": 0, "bf16": 1, "q8_0": 2, "q4_0": 3}
    _KV = {"f32": 0, "f16": 1, "bf16": 2}

    @classmethod
    def new(cls):
        return cls()

    def to_c(self):
        c = CConfig()
        for f in ("hidden_dim", "num_layers", "num_heads", "intermediate_dim", "vocab_size",
                  "max_seq_len", "head_dim", "max_batch"):
            v = int(getattr(self, f))
            if v < 0:
                raise ConfigError(f"Invalid configuration: {f} = {v}: must not be negative")
            setattr(c, f, v)
        c.dropout, c.attention_dropout = self.dropout, self.attention_dropout
        c.layer_norm_eps = self.layer_norm_eps
        c.use_bias = 1 if self.use_bias else 0
        for field, table in (("activation", self._ACT), ("norm", self._NORM),
                             ("norm_scope", self._SCOPE), ("weight_dtype", self._WD),
                             ("kv_dtype", self._KV)):
            v = getattr(self, field)
            if v not in table:
                raise ConfigError(f"Invalid configuration: {field} = {v!r}: unknown value")
            setattr(c, field, table[v])
        return c

    @classmethod
    def from_c(cls, c):
        inv = lambda table: {v: k for k, v in table.items()}
        return cls(hidden_dim=int(c.hidden_dim), num_layers=int(c.num_layers), num_heads=int(c.num_heads),
                   intermediate_dim=int(c.intermediate_dim), vocab_size=int(c.vocab_size),
                   max_seq_len=int(c.max_seq_len), dropout=float(c.dropout),
                   attention_dropout=float(c.attention_dropout), layer_norm_eps=float(c.layer_norm_eps),
                   use_bias=bool(c.use_bias), activation=inv(cls._ACT)[int(c.activation)],
                   norm=inv(cls._NORM)[int(c.norm)], norm_scope=inv(cls._SCOPE)[int(c.norm_scope)],
                   weight_dtype=inv(cls._WD)[int(c.weight_dtype)], kv_dtype=inv(cls._KV)[int(c.kv_dtype)],
                   head_dim=int(c.head_dim), max_batch=max(1, int(c.max_batch)))

    def validate(self):
        """Transformer250MConfig::validate (core/model.rs:487-531)."""
        c = self.to_c()
        _check(_lib.load().coeus_config_validate(C.byref(c)))

    def num_parameters(self):
        """Length of the flat parameter buffer build() allocates (lib.rs:541-580)."""
        c = self.to_c()
        return int(_lib.load().coeus_config_num_parameters(C.byref(c)))

    def used_parameters(self):
        c = self.to_c()
        return int(_lib.load().coeus_config_used_parameters(C.byref(c)))


@dataclass
class BasicGenerationConfig:
    """BasicGenerationConfig (core/model.rs:718-753) with its Default."""

    max_length: int = 100
    temperature: float = 1.0
    top_k: int = None
    top_p: float = None


# ---------------------------------------------------------------- plugin / builder / model
class TransformerModelPlugin:
    """TransformerModelPlugin (lib.rs:503-533)."""

    def id(self):
        return "transformer_model"

    def version(self):
        return (0, 1, 0)

    def capabilities(self):
        return ("model_building", "transformer", "250M_params")

    def create_builder(self):
        return TransformerModelBuilder()


class TransformerModelBuilder:
    """TransformerModelBuilder (lib.rs:537-639)."""

    def build(self, config, parameters=None, seed=None):
        """build(config) (lib.rs:587-638): validates, initialises the flat parameter buffer with
        the reference's deterministic sin init (lib.rs:604-611) and uploads it.

        `parameters` (a flat float32 array in the reference's layout) replaces the default init;
        `seed` asks for synthetic N(0, 0.02)-like weights generated on the device instead."""
        config.validate()
        lib = _lib.load()
        c = config.to_c()
        n_total = int(lib.coeus_config_num_parameters(C.byref(c)))
        handle = C.c_void_p()
        if seed is not None:
            _check(lib.coeus_model_create_seeded(C.byref(c), int(seed), C.byref(handle)))
        else:
            if parameters is None:
                parameters = np.empty(n_total, dtype=np.float32)
                _check(lib.coeus_init_default_parameters(parameters.ctypes.data, n_total,
                                                         config.hidden_dim))
            parameters = np.ascontiguousarray(parameters, dtype=np.float32)
            _check(lib.coeus_model_create(C.byref(c), parameters.ctypes.data, parameters.size,
                                          C.byref(handle)))
        model = TransformerModel(config, handle)
        if seed is None:
            model._parameters = parameters  # kept on the host for write_to, like the reference's Vec<f32>
        return model

    def load(self, path, **overrides):
        """TransformerModel::read_from (lib.rs:1008-1121) on a `.rustllm` file: header, checksummed
        parameters, config from the metadata (fields the file does not name keep their defaults).
        `overrides` replace config fields after reading (e.g. weight_dtype="q4_0")."""
        from .serialization import read_rustllm
        config, parameters = read_rustllm(path)
        for k, v in overrides.items():
            setattr(config, k, v)
        return self.build(config, parameters=parameters)


class TransformerModel:
    """TransformerModel (lib.rs:649-654) with Model (lib.rs:775-785) and ForwardModel
    (lib.rs:787-924)."""

    def __init__(self, config, handle):
        self._config = config
        self._h = handle

    def config(self):
        return self._config

    def name(self):
        return _lib.load().coeus_model_name(self._h).decode()

    def num_parameters(self):
        return int(_lib.load().coeus_model_num_parameters(self._h))

    def weight_bytes(self):
        return int(_lib.load().coeus_model_weight_bytes(self._h))

    def resident_bytes(self):
        """weight_bytes() plus the resident f16 copies that quantised models keep for the prompt pass."""
        return int(_lib.load().coeus_model_resident_bytes(self._h))

    @staticmethod
    def _ids(input_ids):
        ids = np.asarray(input_ids)
        if ids.size and (ids.dtype.kind not in "iu" or (ids.dtype.kind == "i" and ids.min() < 0)):
            raise ProcessingError("Token IDs must be non-negative integers")
        return np.ascontiguousarray(ids, dtype=np.uint64)

    def forward(self, input_ids):
        """forward(Vec<usize>) -> Vec<f32>: logits of the last token (lib.rs:791-919)."""
        ids = self._ids(input_ids).ravel()
        out = np.empty(self._config.vocab_size, dtype=np.float32)
        _check(_lib.load().coeus_model_forward(self._h, ids.ctypes.data, ids.size, out.ctypes.data))
        return out

    def forward_all(self, input_ids):
        """Logits of every row, [seq_len, vocab_size]."""
        ids = self._ids(input_ids).ravel()
        out = np.empty((max(ids.size, 1), self._config.vocab_size), dtype=np.float32)
        _check(_lib.load().coeus_model_forward_all(self._h, ids.ctypes.data, ids.size,
                                                   out.ctypes.data))
        return out

    def generate(self, input_ids, config=None, seed=0):
        """GenerativeModel::generate(input, config) (core/model.rs:138-144): the prompt pass, then
        config.max_length tokens (fewer if max_seq_len ends first), each drawn from the logits of
        the sequence so far.  Returns the generated token ids."""
        config = config or BasicGenerationConfig()
        ids = self._ids(input_ids)
        room = self._config.max_seq_len - ids.size
        n = min(int(config.max_length), room)
        if n <= 0:
            return []
        with_session = self.session(batch=1, max_ctx=ids.size + n)
        try:
            logits = with_session.prefill(ids.reshape(1, -1))
            # the first new token comes from the prompt's last logits, drawn on the device too
            from .device import DeviceArray
            d_logits = DeviceArray.from_host(logits.astype(np.float32))
            d_id = DeviceArray((1,), np.uint64)
            cfg = _lib.CSampling(float(config.temperature), int(config.top_k or 0), float(config.top_p or 0.0), int(seed))
            _check(_lib.load().coeus_op_sample(d_logits.ptr, 1, logits.shape[-1], C.byref(cfg), ids.size,
                                               d_id.ptr, None))
            _check(_lib.load().coeus_device_synchronize())
            first = d_id.to_host()
            out = [int(first[0])]
            if n > 1:
                more = with_session.generate(first, n - 1, config.temperature, config.top_k, config.top_p, seed)
                out += [int(t) for t in more[0]]
            return out
        finally:
            with_session.close()

    def write_to(self, path):
        """ModelSerializable::write_to (lib.rs:931-1006): header, parameters, metadata."""
        from .serialization import write_rustllm
        if getattr(self, "_parameters", None) is None:
            raise ProcessingError("Processing error: this model was generated on the device from a "
                                  "seed; there is no host parameter vector to write")
        write_rustllm(path, self._config, self._parameters)

    def session(self, batch=1, max_ctx=None):
        return Session(self, batch, max_ctx or self._config.max_seq_len)

    def close(self):
        if self._h:
            _lib.load().coeus_model_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Session:
    """KV-cache generation state (an extension: the reference recomputes the whole sequence)."""

    def __init__(self, model, batch, max_ctx):
        self._model = model  # keeps the model alive
        self.batch = batch
        self._h = C.c_void_p()
        _check(_lib.load().coeus_session_create(model._h, batch, max_ctx, C.byref(self._h)))

    def _ids2d(self, ids):
        ids = TransformerModel._ids(ids)
        if ids.ndim == 1:
            ids = ids.reshape(1, -1) if self.batch == 1 else ids.reshape(self.batch, -1)
        if ids.shape[0] != self.batch:
            raise ProcessingError(f"expected ids for {self.batch} sequences, got {ids.shape[0]}")
        return np.ascontiguousarray(ids)

    def prefill(self, ids, want_logits=True):
        ids = self._ids2d(ids)
        V = self._model._config.vocab_size
        out = np.empty((self.batch, V), dtype=np.float32) if want_logits else None
        _check(_lib.load().coeus_session_prefill(self._h, ids.ctypes.data, ids.shape[1],
                                                 out.ctypes.data if want_logits else None))
        return out

    def decode(self, ids):
        ids = TransformerModel._ids(ids).ravel()
        if ids.size != self.batch:
            raise ProcessingError(f"expected {self.batch} ids, got {ids.size}")
        out = np.empty((self.batch, self._model._config.vocab_size), dtype=np.float32)
        _check(_lib.load().coeus_session_decode(self._h, ids.ctypes.data, out.ctypes.data))
        return out

    def decode_greedy(self, first_ids, n_steps):
        ids = TransformerModel._ids(first_ids).ravel()
        if ids.size != self.batch:
            raise ProcessingError(f"expected {self.batch} ids, got {ids.size}")
        out = np.empty((self.batch, max(int(n_steps), 1)), dtype=np.uint64)
        _check(_lib.load().coeus_session_decode_greedy(self._h, ids.ctypes.data, int(n_steps),
                                                       out.ctypes.data))
        return out

    def generate(self, first_ids, n_steps, temperature=1.0, top_k=None, top_p=None, seed=0):
        """n_steps tokens per sequence drawn on the device (coeus_session_generate): the inner loop
        of GenerativeModel::generate with a BasicGenerationConfig's temperature / top_k / top_p."""
        first = np.ascontiguousarray(first_ids, dtype=np.uint64).reshape(self.batch)
        out = np.empty((self.batch, int(n_steps)), dtype=np.uint64)
        cfg = _lib.CSampling(float(temperature), int(top_k or 0), float(top_p or 0.0), int(seed))
        _check(_lib.load().coeus_session_generate(self._h, first.ctypes.data, int(n_steps), C.byref(cfg),
                                                  out.ctypes.data))
        return out

    def set_graph(self, enabled):
        _check(_lib.load().coeus_session_set_graph(self._h, 1 if enabled else 0))

    @property
    def graph_enabled(self):
        """False when greedy decoding and the timing hooks launch kernel by kernel: switched off
        with set_graph(False), or a profiler tool library is loaded in the process."""
        return bool(_lib.load().coeus_session_graph_enabled(self._h))

    def time_decode_matmuls(self, reps):
        """Returns (milliseconds, launches, algorithmic_bytes) for `reps` replays of the decode
        matmuls of one step (see coeus_session_time_decode_matmuls)."""
        ms, n, b = C.c_float(), C.c_uint64(), C.c_uint64()
        _check(_lib.load().coeus_session_time_decode_matmuls(self._h, int(reps), C.byref(ms),
                                                             C.byref(n), C.byref(b)))
        return ms.value, n.value, b.value

    def time_decode_attention(self, reps):
        """The same for the attention launches of one step at the current context length."""
        ms, n, b = C.c_float(), C.c_uint64(), C.c_uint64()
        _check(_lib.load().coeus_session_time_decode_attention(self._h, int(reps), C.byref(ms),
                                                               C.byref(n), C.byref(b)))
        return ms.value, n.value, b.value

    @property
    def position(self):
        return int(_lib.load().coeus_session_position(self._h))

    def reset(self):
        _check(_lib.load().coeus_session_reset(self._h))

    def close(self):
        if self._h:
            _lib.load().coeus_session_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
