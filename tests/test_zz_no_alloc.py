"""coeus_op_attention_decode_static: the decode attention whose partial records and arrival
counters live in a static device array (no device allocation in the call), against
coeus_op_attention_decode, which allocates them per call.  Same kernels, same record order, so the
outputs must be identical bit for bit.  Two calls in a row, the second with a smaller input: the
array keeps the first call's records and counters, which the second must not see."""
import numpy as np
import pytest

from coeus_amd import _lib
from coeus_amd.device import DeviceArray, synchronize
from coeus_amd.plugin import ProcessingError, _check
from gpu_util import dev

pytestmark = pytest.mark.gpu


def _case(rng, batch, heads, hd, max_ctx):
    inner = heads * hd
    qkv = rng.standard_normal((batch, 3 * inner)).astype(np.float32)
    k = rng.standard_normal((batch, heads, max_ctx, hd)).astype(np.float16)
    v = rng.standard_normal((batch, heads, max_ctx, hd)).astype(np.float16)
    return dev(qkv), dev(k.view(np.uint16)), dev(v.view(np.uint16))


@pytest.mark.parametrize("merge", [_lib.MERGE_IN_KERNEL, _lib.MERGE_SEPARATE])
def test_static_scratch_equals_allocating_entry_point(merge):
    lib = _lib.load()
    rng = np.random.default_rng(5)
    # (batch, heads, head_dim, max_ctx, ctx, nsplit): large first, then smaller in every dimension
    calls = [(4, 32, 128, 2048, 2048, 16), (1, 6, 64, 1024, 700, 5), (2, 32, 128, 2048, 1500, 16)]
    for batch, heads, hd, max_ctx, ctx, nsplit in calls:
        dq, dk, dv = _case(rng, batch, heads, hd, max_ctx)
        want, got = DeviceArray((batch, heads * hd), np.float32), DeviceArray((batch, heads * hd), np.float32)
        want.zero_()
        got.zero_()
        _check(lib.coeus_op_attention_decode(dq.ptr, dk.ptr, dv.ptr, _lib.KV_F16, batch, heads, hd, max_ctx, ctx,
                                             nsplit, merge, want.ptr, None))
        _check(lib.coeus_op_attention_decode_static(dq.ptr, dk.ptr, dv.ptr, _lib.KV_F16, batch, heads, hd, max_ctx,
                                                    ctx, nsplit, merge, got.ptr, None))
        synchronize()
        w, g = want.to_host(), got.to_host()
        assert np.isfinite(w).all() and np.abs(w).max() > 0
        assert np.array_equal(w.view(np.uint32), g.view(np.uint32)), (batch, heads, hd, ctx, nsplit)
        for a in (dq, dk, dv, want, got):
            a.free()


def test_static_scratch_limits():
    lib = _lib.load()
    d = DeviceArray((16,), np.float32)
    # 16 x 32 x 16 = 8192 records > 4096; 40 x 32 = 1280 pairs > 1024
    for batch, heads, nsplit in [(16, 32, 16), (40, 32, 1)]:
        with pytest.raises(ProcessingError, match="static buffer holds"):
            _check(lib.coeus_op_attention_decode_static(d.ptr, d.ptr, d.ptr, _lib.KV_F16, batch, heads, 128, 4096, 4096,
                                                        nsplit, 0, d.ptr, None))
