"""Helpers for the GPU tests: device buffers and the kernels both go through the C ABI."""
import ctypes as C

import numpy as np

from coeus_amd import _lib
from coeus_amd.device import DeviceArray, synchronize
from coeus_amd.plugin import _check


def dev(a, dtype=None):
    return DeviceArray.from_host(a, dtype)


class Weight:
    """coeus_weight handle (a linear weight resident on the device)."""

    def __init__(self, dtype, w_kn=None, seed=None, base=0, shape=None):
        self.lib = _lib.load()
        self.h = C.c_void_p()
        if w_kn is not None:
            w = np.ascontiguousarray(w_kn, dtype=np.float32)
            self.k, self.n = w.shape
            _check(self.lib.coeus_weight_create(dtype, w.ctypes.data, self.k, self.n, C.byref(self.h)))
        else:
            self.k, self.n = shape
            _check(self.lib.coeus_weight_create_seeded(dtype, seed, base, self.k, self.n, C.byref(self.h)))

    def dequantize(self):
        out = np.empty((self.k, self.n), dtype=np.float32)
        _check(self.lib.coeus_weight_dequantize(self.h, out.ctypes.data))
        return out

    def bytes(self):
        return int(self.lib.coeus_weight_bytes(self.h))

    def gemv(self, x, bias=None, residual=None, epilogue=0, stream=None):
        batch = x.shape[0]
        n_eff = self.n // 2 if epilogue == _lib.EPI_SILU_GATE else self.n
        y = DeviceArray((batch, n_eff), np.float32)
        _check(self.lib.coeus_op_gemv(self.h, x.ptr, batch,
                                      bias.ptr if bias is not None else None,
                                      residual.ptr if residual is not None else None,
                                      epilogue, y.ptr, stream))
        synchronize()
        return y.to_host()

    def gemm(self, a, bias=None, residual=None, epilogue=0, stream=None):
        m = a.shape[0]
        n_eff = self.n // 2 if epilogue == _lib.EPI_SILU_GATE else self.n
        c = DeviceArray((m, n_eff), np.float32)
        _check(self.lib.coeus_op_gemm(self.h, a.ptr, m,
                                      bias.ptr if bias is not None else None,
                                      residual.ptr if residual is not None else None,
                                      epilogue, c.ptr, stream))
        synchronize()
        return c.to_host()

    def close(self):
        if self.h:
            self.lib.coeus_weight_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def oracle_roundtrip(orc, dtype, w_kn):
    """What the device must hold for a [k, n] matrix: blocks run along k per output column."""
    w = np.ascontiguousarray(w_kn, dtype=np.float32)
    if dtype == _lib.W_F32:
        return w
    if dtype == _lib.W_BF16:
        return orc.bf16_round(w)
    quant, deq = ((orc.quantize_q8_0, orc.dequantize_q8_0) if dtype == _lib.W_Q8_0 else
                  (orc.quantize_q4_0, orc.dequantize_q4_0))
    wt = np.ascontiguousarray(w.T)  # [n, k]: each row is one output's reduction run
    q, d = quant(wt)
    return np.ascontiguousarray(deq(q, d).reshape(wt.shape).T)


def rel_err(got, want):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    return np.abs(got - want).max() / max(np.abs(want).max(), 1e-30)
