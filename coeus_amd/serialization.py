"""`.rustllm` model files (the reference's core/serialization.rs + TransformerModel's
ModelSerializable impl, lib.rs:930-1121), through the C ABI's coeus_rustllm_* functions."""
import ctypes as C
import os

import numpy as np

from . import _lib
from ._lib import CConfig
from .plugin import Transformer250MConfig, _check


def checksum(parameters):
    """calculate_checksum (core/serialization.rs:375-385): rotate-add over the f32 bit patterns."""
    p = np.ascontiguousarray(parameters, dtype=np.float32)
    return int(_lib.load().coeus_rustllm_checksum(p.ctypes.data, p.size))


def write_rustllm(path, config, parameters):
    p = np.ascontiguousarray(parameters, dtype=np.float32)
    c = config.to_c()
    _check(_lib.load().coeus_rustllm_write(os.fsencode(path), C.byref(c), p.ctypes.data, p.size))


def read_rustllm(path):
    """Returns (Transformer250MConfig, flat float32 parameter array)."""
    lib = _lib.load()
    c, n = CConfig(), C.c_uint64()
    _check(lib.coeus_rustllm_read_header(os.fsencode(path), C.byref(c), C.byref(n)))
    params = np.empty(n.value, dtype=np.float32)
    _check(lib.coeus_rustllm_read_parameters(os.fsencode(path), params.ctypes.data, n.value))
    return Transformer250MConfig.from_c(c), params
