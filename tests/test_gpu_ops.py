"""GPU parity of the individual HIP kernels, through the C ABI, against the CPU oracle.

Bars: bit-exact for integer/byte work (quantisation, dequantisation, the synthetic generator);
max-abs relative 1e-3 for f32 arithmetic and 2e-2 for bf16/quantised arithmetic (the kernels
round activations to f16/bf16 for the matrix cores); tighter figures below are what the kernels
actually achieve against a float64 product of the SAME rounded operands."""
import ctypes as C

import numpy as np
import pytest

from coeus_amd import _lib
from coeus_amd.plugin import _check
from coeus_amd.device import DeviceArray, synchronize
from gpu_util import Weight, dev, oracle_roundtrip, rel_err

pytestmark = pytest.mark.gpu

DT = {"f32": _lib.W_F32, "bf16": _lib.W_BF16, "q8_0": _lib.W_Q8_0, "q4_0": _lib.W_Q4_0}


def _f16(x):
    return x.astype(np.float16).astype(np.float64)


def test_device_is_gfx950():
    lib = _lib.load()
    name = C.create_string_buffer(256)
    hbm, cus = C.c_uint64(), C.c_uint32()
    _check(lib.coeus_device_info(name, 256, C.byref(hbm), C.byref(cus)))
    print("device:", name.value.decode(), hbm.value >> 30, "GiB", cus.value, "CUs", flush=True)
    assert b"gfx950" in name.value


@pytest.mark.parametrize("dtype", ["f32", "bf16", "q8_0", "q4_0"])
@pytest.mark.parametrize("shape", [(128, 16), (256, 48), (96, 50), (768, 130)])
def test_weight_conversion_is_bit_exact(orc, dtype, shape):
    k, n = shape
    rng = np.random.default_rng(k * 1000 + n)
    w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    w[32:64, 3] = 0  # an all-zero block
    wt = Weight(DT[dtype], w)
    got = wt.dequantize()
    want = oracle_roundtrip(orc, DT[dtype], w)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_seeded_weight_matches_cpu_generator(orc):
    k, n, seed, base = 64, 40, 0xC0E05, 123_456_789_012
    wt = Weight(_lib.W_F32, seed=seed, base=base, shape=(k, n))
    got = wt.dequantize()
    L = orc.lib()
    want = np.array([[np.float32(0.02) * np.float32(L.orc_synth_normal(seed, base + l * n + j))
                      for j in range(n)] for l in range(k)], dtype=np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # the quantised form of a seeded weight equals quantising those values on the CPU
    wq = Weight(_lib.W_Q4_0, seed=seed, base=base, shape=(k, n))
    assert np.array_equal(wq.dequantize(), oracle_roundtrip(orc, _lib.W_Q4_0, want))


@pytest.mark.parametrize("dtype", ["f32", "bf16", "q8_0", "q4_0"])
# (17408, 48, 2): 34 quads of 512 k, more than 16 waves x 2 take in one pass of the quantised kernel
@pytest.mark.parametrize("k,n,batch", [(128, 16, 1), (256, 50, 3), (768, 3072, 1), (3072, 768, 8),
                                       (96, 33, 16), (4096, 512, 2), (17408, 48, 2)])
def test_gemv(orc, dtype, k, n, batch):
    rng = np.random.default_rng(k + n + batch)
    w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    x = rng.standard_normal((batch, k)).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32) * 0.1
    res = rng.standard_normal((batch, n)).astype(np.float32)
    wt = Weight(DT[dtype], w)
    wdq = oracle_roundtrip(orc, DT[dtype], w).astype(np.float64)
    quant = dtype in ("q8_0", "q4_0")
    xr = _f16(x) if quant else x.astype(np.float64)
    # plain product
    y = wt.gemv(dev(x))
    assert rel_err(y, xr @ wdq) < 2e-5          # kernel arithmetic on the rounded operands
    assert rel_err(y, x.astype(np.float64) @ wdq) < (2e-2 if quant else 1e-3)
    # bias + GELU + residual epilogue (MT:348-358, MT:494-496 fused)
    y2 = wt.gemv(dev(x), bias=dev(bias), residual=dev(res), epilogue=_lib.EPI_GELU)
    pre = xr @ wdq + bias
    want2 = 0.5 * pre * (1 + np.tanh(0.7978845608028654 * pre * (1 + 0.044715 * pre * pre))) + res
    assert rel_err(y2, want2) < 2e-5
    # results for a row do not depend on the batch it travels in: bit for bit among batches of up
    # to 4 and among larger ones (the quantised decode matmul has one kernel for each range, which
    # sum the blocks of a row in different orders), to rounding between the two
    y1 = wt.gemv(dev(x[:1]))
    same_kernel = batch <= 4 or not quant
    assert (np.array_equal(y1[0], y[0]) if same_kernel and quant else rel_err(y1[0], y[0]) < (2e-5 if quant else 1e-6))
    if quant and batch > 4:
        y5 = wt.gemv(dev(x[:5]))
        assert np.array_equal(y5[0], y[0])


@pytest.mark.parametrize("dtype", ["f32", "bf16", "q4_0"])
def test_gemv_gated_epilogue(orc, dtype):
    rng = np.random.default_rng(77)
    k, n_eff, batch = 256, 88, 5
    w = (rng.standard_normal((k, 2 * n_eff)) * 0.05).astype(np.float32)  # columns (gate_m, up_m)
    x = rng.standard_normal((batch, k)).astype(np.float32)
    bias = (rng.standard_normal(2 * n_eff) * 0.1).astype(np.float32)
    wt = Weight(DT[dtype], w)
    wdq = oracle_roundtrip(orc, DT[dtype], w).astype(np.float64)
    xr = _f16(x) if dtype == "q4_0" else x.astype(np.float64)
    pre = xr @ wdq + bias
    g, u = pre[:, 0::2], pre[:, 1::2]
    want = g / (1 + np.exp(-g)) * u
    y = wt.gemv(dev(x), bias=dev(bias), epilogue=_lib.EPI_SILU_GATE)
    assert y.shape == (batch, n_eff) and rel_err(y, want) < 2e-5


@pytest.mark.parametrize("dtype", ["f32", "bf16", "q8_0", "q4_0"])
@pytest.mark.parametrize("m,k,n", [(1, 64, 16), (37, 96, 50), (128, 768, 768), (200, 256, 333),
                                   (130, 3072, 768)])
def test_gemm(orc, dtype, m, k, n):
    rng = np.random.default_rng(m + k + n)
    w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    a = rng.standard_normal((m, k)).astype(np.float32)
    bias = (rng.standard_normal(n) * 0.1).astype(np.float32)
    res = rng.standard_normal((m, n)).astype(np.float32)
    wt = Weight(DT[dtype], w)
    wdq = oracle_roundtrip(orc, DT[dtype], w)
    if dtype == "f32":
        ar, wr, tol = a.astype(np.float64), wdq.astype(np.float64), 2e-5
        # the oracle's own matmul (MT:50-74) on the same operands
        assert rel_err(wt.gemm(dev(a)), orc.matmul(a, w)) < 1e-5
    elif dtype == "bf16":
        ar, wr, tol = orc.bf16_round(a).astype(np.float64), wdq.astype(np.float64), 2e-5
    else:
        ar, wr, tol = _f16(a), _f16(wdq), 2e-5  # prefill uses f16-rounded dequantised weights
    c = wt.gemm(dev(a))
    assert rel_err(c, ar @ wr) < tol
    assert rel_err(c, a.astype(np.float64) @ wdq.astype(np.float64)) < (1e-3 if dtype == "f32" else 2e-2)
    c2 = wt.gemm(dev(a), bias=dev(bias), residual=dev(res), epilogue=_lib.EPI_GELU)
    pre = ar @ wr + bias
    want2 = 0.5 * pre * (1 + np.tanh(0.7978845608028654 * pre * (1 + 0.044715 * pre * pre))) + res
    assert rel_err(c2, want2) < tol


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_gemm_gated_epilogue(orc, dtype):
    rng = np.random.default_rng(78)
    m, k, n_eff = 70, 128, 72
    w = (rng.standard_normal((k, 2 * n_eff)) * 0.05).astype(np.float32)
    a = rng.standard_normal((m, k)).astype(np.float32)
    wt = Weight(DT[dtype], w)
    ar = a.astype(np.float64) if dtype == "f32" else orc.bf16_round(a).astype(np.float64)
    pre = ar @ oracle_roundtrip(orc, DT[dtype], w).astype(np.float64)
    g, u = pre[:, 0::2], pre[:, 1::2]
    c = wt.gemm(dev(a), epilogue=_lib.EPI_SILU_GATE)
    assert c.shape == (m, n_eff) and rel_err(c, g / (1 + np.exp(-g)) * u) < 2e-5


@pytest.mark.parametrize("dtype", ["bf16", "q8_0"])
def test_gemm_gelu_fast_epilogue_walks(orc, dtype):
    """GELU without a residual on a launch of more than 128 full tiles (132 tiles of 256 x 256, so
    nothing is split along k): the prompt matmul's row walk, which evaluates the tanh form of
    math::gelu (MT:94-99) through the hardware exponential and reciprocal.  With and without a
    bias, f32 output, against float64 tanh-GELU on the rounded operands at the operator bar."""
    rng = np.random.default_rng(4242)
    m, k, n = 2816, 128, 3072
    w = (rng.standard_normal((k, n)) * 0.2).astype(np.float32)   # pre-activations of a few units:
    a = rng.standard_normal((m, k)).astype(np.float32)           # both tails of the tanh are hit
    bias = rng.standard_normal(n).astype(np.float32)
    wt = Weight(DT[dtype], w)
    wdq = oracle_roundtrip(orc, DT[dtype], w)
    if dtype == "bf16":
        ar, wr = orc.bf16_round(a).astype(np.float64), wdq.astype(np.float64)
    else:
        ar, wr = _f16(a), _f16(wdq)
    gelu = lambda x: 0.5 * x * (1 + np.tanh(0.7978845608028654 * x * (1 + 0.044715 * x * x)))
    pre = ar @ wr
    assert np.abs(pre).max() > 6  # saturated on both sides
    assert rel_err(wt.gemm(dev(a), epilogue=_lib.EPI_GELU), gelu(pre)) < 2e-5
    assert rel_err(wt.gemm(dev(a), bias=dev(bias), epilogue=_lib.EPI_GELU), gelu(pre + bias)) < 2e-5


@pytest.mark.parametrize("dtype", ["bf16", "q4_0", "f32"])
@pytest.mark.parametrize("m,k,n", [(70, 1024, 334), (300, 2048, 520), (16, 4096, 256)])
def test_gemm_split_along_k(orc, dtype, m, k, n):
    """Few output tiles and a long k: the 16-bit matmul runs as several workgroups per tile over
    shares of k plus a kernel that sums the partial products and applies the epilogue (here 4, 8
    and 16 shares; 334 and 520 columns end inside a tile, 334 is not a multiple of 4).  Plain,
    bias + GELU + residual, and gated epilogues against float64 on the rounded operands.  The f32
    matmul splits its 32x32-tile launches from 1536 elements of k (here 5 and 8 shares; the first
    shape runs unsplit)."""
    rng = np.random.default_rng(m * 7 + k + n)
    w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    a = rng.standard_normal((m, k)).astype(np.float32)
    bias = (rng.standard_normal(n) * 0.1).astype(np.float32)
    res = rng.standard_normal((m, n)).astype(np.float32)
    wt = Weight(DT[dtype], w)
    wdq = oracle_roundtrip(orc, DT[dtype], w)
    if dtype == "bf16":
        ar, wr = orc.bf16_round(a).astype(np.float64), wdq.astype(np.float64)
    elif dtype == "f32":
        ar, wr = a.astype(np.float64), w.astype(np.float64)
    else:
        ar, wr = _f16(a), _f16(wdq)
    pre = ar @ wr
    assert rel_err(wt.gemm(dev(a)), pre) < 2e-5
    c2 = wt.gemm(dev(a), bias=dev(bias), residual=dev(res), epilogue=_lib.EPI_GELU)
    pb = pre + bias
    want2 = 0.5 * pb * (1 + np.tanh(0.7978845608028654 * pb * (1 + 0.044715 * pb * pb))) + res
    assert rel_err(c2, want2) < 2e-5
    g, u = pre[:, 0::2], pre[:, 1::2]
    c3 = wt.gemm(dev(a), epilogue=_lib.EPI_SILU_GATE)
    assert c3.shape == (m, n // 2) and rel_err(c3, g / (1 + np.exp(-g)) * u) < 2e-5
    # the sum over the shares runs in a fixed order: the same call gives the same bits
    assert np.array_equal(wt.gemm(dev(a)), wt.gemm(dev(a)))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["bf16", "q8_0"])
@pytest.mark.parametrize("k", [64, 128, 192, 256, 320, 576])
def test_gemm_slice_pipeline_boundaries(orc, dtype, k):
    """The 16-bit matmul for k % 64 == 0 keeps three slices of A rows and two of W rows in LDS and
    changes its schedule with the number of 64-wide slices (1, 2, 3: nothing left to request; from 4
    on the steady-state period runs).  300 rows and 392 columns end inside the second tiles, no
    launch here is split along k.  Plain, bias + GELU + residual, and gated epilogues against
    float64 on the rounded operands."""
    m, n = 300, 392
    rng = np.random.default_rng(k + 5)
    w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    a = rng.standard_normal((m, k)).astype(np.float32)
    bias = (rng.standard_normal(n) * 0.1).astype(np.float32)
    res = rng.standard_normal((m, n)).astype(np.float32)
    wt = Weight(DT[dtype], w)
    wdq = oracle_roundtrip(orc, DT[dtype], w)
    if dtype == "bf16":
        ar, wr = orc.bf16_round(a).astype(np.float64), wdq.astype(np.float64)
    else:
        ar, wr = _f16(a), _f16(wdq)
    pre = ar @ wr
    assert rel_err(wt.gemm(dev(a)), pre) < 2e-5
    c2 = wt.gemm(dev(a), bias=dev(bias), residual=dev(res), epilogue=_lib.EPI_GELU)
    pb = pre + bias
    want2 = 0.5 * pb * (1 + np.tanh(0.7978845608028654 * pb * (1 + 0.044715 * pb * pb))) + res
    assert rel_err(c2, want2) < 2e-5
    g, u = pre[:, 0::2], pre[:, 1::2]
    c3 = wt.gemm(dev(a), epilogue=_lib.EPI_SILU_GATE)
    assert c3.shape == (m, n // 2) and rel_err(c3, g / (1 + np.exp(-g)) * u) < 2e-5


@pytest.mark.parametrize("dtype,m,k,n", [("bf16", 4100, 512, 4090), ("q8_0", 4024, 1024, 4360)])
def test_gemm_last_round_split(orc, dtype, m, k, n):
    """More than 256 output tiles with a short last round (17 x 16 = 256 + 16 and 16 x 18 = 256 +
    32 tiles): only the tiles of that round are split along k, through private partial tiles.  Rows
    and columns end inside the last tiles; 4090 is not a multiple of 4."""
    rng = np.random.default_rng(m + k + n)
    w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    a = rng.standard_normal((m, k)).astype(np.float32)
    bias = (rng.standard_normal(n) * 0.1).astype(np.float32)
    res = rng.standard_normal((m, n)).astype(np.float32)
    wt = Weight(DT[dtype], w)
    wdq = oracle_roundtrip(orc, DT[dtype], w)
    if dtype == "bf16":
        ar, wr = orc.bf16_round(a).astype(np.float64), wdq.astype(np.float64)
    else:
        ar, wr = _f16(a), _f16(wdq)
    pre = ar @ wr
    da = dev(a)
    assert rel_err(wt.gemm(da), pre) < 2e-5
    c2 = wt.gemm(da, bias=dev(bias), residual=dev(res), epilogue=_lib.EPI_GELU)
    pb = pre + bias
    want2 = 0.5 * pb * (1 + np.tanh(0.7978845608028654 * pb * (1 + 0.044715 * pb * pb))) + res
    assert rel_err(c2, want2) < 2e-5
    g, u = pre[:, 0::2], pre[:, 1::2]
    c3 = wt.gemm(da, epilogue=_lib.EPI_SILU_GATE)
    assert c3.shape == (m, n // 2) and rel_err(c3, g / (1 + np.exp(-g)) * u) < 2e-5
    # the shares are summed in a fixed order: two calls agree bit for bit
    assert np.array_equal(wt.gemm(da), wt.gemm(da))


@pytest.mark.parametrize("dtype", ["q4_0", "q8_0"])
@pytest.mark.parametrize("m,k,n", [(1, 2048, 2048), (16, 4096, 1030), (33, 2048, 2064), (64, 1024, 4098)])
def test_gemm_short_prompt_on_quantised_weights(orc, dtype, m, k, n):
    """Up to 64 rows on a quantised matrix of at least 4 M weights: the matmul that streams the
    quantised blocks (two and four fragments of 16 rows; 1030, 2064 and 4098 columns end inside a
    tile of 16 / a group of 128 weight rows; every launch here is split along k).  Its weights are
    f16(q * d), the values of the f16 copies that longer prompts multiply with, so the same
    float64 reference and bar apply."""
    rng = np.random.default_rng(m * 11 + k + n)
    w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    a = rng.standard_normal((m, k)).astype(np.float32)
    bias = (rng.standard_normal(n) * 0.1).astype(np.float32)
    res = rng.standard_normal((m, n)).astype(np.float32)
    wt = Weight(DT[dtype], w)
    ar, wr = _f16(a), _f16(oracle_roundtrip(orc, DT[dtype], w))
    pre = ar @ wr
    da = dev(a)
    assert rel_err(wt.gemm(da), pre) < 2e-5
    c2 = wt.gemm(da, bias=dev(bias), residual=dev(res), epilogue=_lib.EPI_GELU)
    pb = pre + bias
    want2 = 0.5 * pb * (1 + np.tanh(0.7978845608028654 * pb * (1 + 0.044715 * pb * pb))) + res
    assert rel_err(c2, want2) < 2e-5
    g, u = pre[:, 0::2], pre[:, 1::2]
    c3 = wt.gemm(da, epilogue=_lib.EPI_SILU_GATE)
    assert c3.shape == (m, n // 2) and rel_err(c3, g / (1 + np.exp(-g)) * u) < 2e-5
    assert np.array_equal(wt.gemm(da), wt.gemm(da))


# (128, 768) and (1031, 770) are large enough for the whole-slice statistics to be reduced by
# many workgroups (the second with a ragged last chunk)
# from 512 rows of at most 1024 elements (a multiple of 4) the per-token norms run one wave per row, with
# 1 / 2 / 4 pieces per lane: (1025, 200), (514, 512), (600, 768); longer rows stay with the row kernel
@pytest.mark.parametrize("rows,hidden", [(1, 768), (7, 48), (128, 768), (3, 4096), (1031, 770), (1025, 200),
                                         (514, 512), (600, 768), (513, 2048), (515, 4096), (512, 4100)])
def test_norm(orc, rows, hidden):
    lib = _lib.load()
    rng = np.random.default_rng(rows + hidden)
    x = (rng.standard_normal((rows, hidden)) * 2 + 0.5).astype(np.float32)
    sc = rng.standard_normal(hidden).astype(np.float32)
    bi = rng.standard_normal(hidden).astype(np.float32)
    dx, ds, db = dev(x), dev(sc), dev(bi)
    y = DeviceArray((rows, hidden), np.float32)
    # reference mode: one mean/variance for the whole slice (MT:105-128)
    _check(lib.coeus_op_norm(0, 0, dx.ptr, rows, hidden, ds.ptr, db.ptr, 1e-5,
                             y.ptr, None))
    synchronize()
    want = orc.layer_norm(x.ravel(), sc, bi, 1e-5).reshape(rows, hidden)
    # The reference accumulates its whole-slice statistics sequentially in f32; over 200-800 k
    # elements that drifts 2e-4 away from the exact value, which the kernel (f64 sums) delivers.
    # Small slices agree tightly with the reference's arithmetic, the large one with the exact
    # statistics, and with the reference's within the f32 bar of 1e-3.
    big = rows * hidden > 100000
    assert rel_err(y.to_host(), want) < (1e-3 if big else 1e-5)
    x64 = x.astype(np.float64)
    exact = sc * (x64 - x64.mean()) / np.sqrt(x64.var() + np.float64(np.float32(1e-5))) + bi
    assert rel_err(y.to_host(), exact) < (2e-6 if big else 1e-5)
    # per-token statistics
    _check(lib.coeus_op_norm(0, 1, dx.ptr, rows, hidden, ds.ptr, db.ptr, 1e-5,
                             y.ptr, None))
    synchronize()
    want_tok = np.stack([orc.layer_norm(x[r], sc, bi, 1e-5) for r in range(rows)])
    assert rel_err(y.to_host(), want_tok) < 1e-5
    # RMSNorm per token
    _check(lib.coeus_op_norm(1, 1, dx.ptr, rows, hidden, ds.ptr, None, 1e-5,
                             y.ptr, None))
    synchronize()
    want_rms = sc * x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + np.float64(np.float32(1e-5)))
    assert rel_err(y.to_host(), want_rms) < 1e-5
    # RMSNorm with one mean square for the whole slice
    _check(lib.coeus_op_norm(1, 0, dx.ptr, rows, hidden, ds.ptr, None, 1e-5,
                             y.ptr, None))
    synchronize()
    want_rms_seq = sc * x64 / np.sqrt((x64 ** 2).mean() + np.float64(np.float32(1e-5)))
    assert rel_err(y.to_host(), want_rms_seq) < 1e-5


def test_norm_whole_slice_far_from_zero(orc):
    """Whole-slice statistics of values whose mean is 2000 standard deviations from zero: the two-launch
    kernel sums x - x[0] and its square in f64, so the variance comes out to f32 rounding where
    sum x^2 - n mean^2 taken from zero would lose five digits."""
    lib = _lib.load()
    rows, hidden = 128, 768
    rng = np.random.default_rng(11)
    x = (1000.0 + 0.5 * rng.standard_normal((rows, hidden))).astype(np.float32)
    sc = rng.standard_normal(hidden).astype(np.float32)
    bi = rng.standard_normal(hidden).astype(np.float32)
    dx, ds, db = dev(x), dev(sc), dev(bi)
    y = DeviceArray((rows, hidden), np.float32)
    x64 = x.astype(np.float64)
    for kind in (0, 1):
        _check(lib.coeus_op_norm(kind, 0, dx.ptr, rows, hidden, ds.ptr, db.ptr if kind == 0 else None, 1e-5, y.ptr, None))
        synchronize()
        eps = np.float64(np.float32(1e-5))
        if kind == 0:
            # the mean is rounded to f32 before it is subtracted, in the reference and here
            mean32 = np.float64(np.float32(x64.mean()))
            want = sc * (x64 - mean32) / np.sqrt(x64.var() + eps) + bi
        else:
            want = sc * x64 / np.sqrt((x64 ** 2).mean() + eps)
        assert rel_err(y.to_host(), want) < 2e-6


def test_embed_and_positional_encoding(orc):
    lib = _lib.load()
    V, H, S, pos0 = 97, 48, 9, 5
    rng = np.random.default_rng(5)
    table = rng.standard_normal((V, H)).astype(np.float32)
    pe = np.empty((32, H), dtype=np.float32)
    _check(lib.coeus_positional_encoding(32, H, pe.ctypes.data))
    assert np.array_equal(pe, orc.positional_encoding(32, H))  # same libm, same bits (MT:398-407)
    ids = rng.integers(0, V, S).astype(np.uint64)
    dt, dp = dev(table), dev(pe)
    dids = dev(ids)
    x = DeviceArray((S, H), np.float32)
    _check(lib.coeus_op_embed(dt.ptr, dp.ptr, dids.ptr, S, pos0, H, x.ptr, None))
    synchronize()
    want = table[ids.astype(np.int64)] + pe[pos0:pos0 + S]  # MT:812-835
    assert np.array_equal(x.to_host(), want)


# (8 and 16 heads: with a multiple of 8 heads the matrix-core kernels renumber their workgroups so
# that a head's query tiles share an XCD; 300 and 260 rows are three query tiles)
@pytest.mark.parametrize("rows,heads,hd", [(3, 2, 4), (19, 4, 12), (128, 12, 64), (70, 2, 128), (300, 3, 64), (257, 2, 128),
                                           (300, 8, 64), (260, 16, 128)])
def test_attention(orc, rows, heads, hd):
    lib = _lib.load()
    rng = np.random.default_rng(rows * heads + hd)
    inner = heads * hd
    qkv = rng.standard_normal((rows, 3 * inner)).astype(np.float32)
    out_d = DeviceArray((rows, inner), np.float32)
    dq = dev(qkv)
    _check(lib.coeus_op_attention(dq.ptr, rows, heads, hd, out_d.ptr, None))
    synchronize()
    out = out_d.to_host()
    q, k, v = (qkv[:, i * inner:(i + 1) * inner].astype(np.float64) for i in range(3))
    want = np.zeros((rows, inner))
    causal = np.tril(np.ones((rows, rows), dtype=bool))
    for h in range(heads):
        sl = slice(h * hd, (h + 1) * hd)
        sc = np.where(causal, q[:, sl] @ k[:, sl].T / np.sqrt(hd), -np.inf)
        p = np.exp(sc - sc.max(-1, keepdims=True))
        want[:, sl] = (p / p.sum(-1, keepdims=True)) @ v[:, sl]
    assert rel_err(out, want) < 1e-5
    # the oracle's MHA (MT:167-300) with identity projections isolates MT:219-278
    eye = np.concatenate([np.eye(inner, dtype=np.float32).ravel()] * 4)
    ref = orc.mha_forward(inner, heads, qkv[:, :inner], qkv[:, inner:2 * inner], qkv[:, 2 * inner:],
                          eye, None, orc.causal_mask(rows), rows).reshape(rows, inner)
    assert rel_err(out, ref) < 1e-5
    # row 0 attends to itself only
    assert rel_err(out[0], v[0]) < 1e-6


# ------------------------------------------------------------------ the decode matmul at the benchmark shapes
# Every instantiation of the quantised decode matmul that the 7B / 1B decode steps launch, at its
# real (k, n), against float64 on the oracle-dequantised weights and f16-rounded activations.

def _seeded(dtype, k, n, seed):
    wt = Weight(DT[dtype], seed=seed, base=0, shape=(k, n))
    return wt, wt.dequantize().astype(np.float64)


REAL_SHAPES = [(4096, 12288, False), (4096, 4096, False), (4096, 22016, True), (11008, 4096, False),
               (4096, 32000, False), (2048, 8192, False), (8192, 2048, False),
               # four tiles per workgroup at batch 16 with a partial last pass over k (35 chunks for
               # 16 waves) and a last workgroup with one real tile of its four
               (4480, 12300, False)]


@pytest.mark.parametrize("dtype", ["q4_0", "q8_0"])
@pytest.mark.parametrize("k,n,gated", REAL_SHAPES)
def test_gemv_benchmark_shapes(orc, dtype, k, n, gated):
    """coeus_op_gemv (activations staged from the f16 interchange buffer): batch 1, 4, 8 and 16 take
    the variants with 1 / 4 / 4 / 4 live accumulator rows, the (11008, 4096) matrix the one with six
    chunks in flight per wave, batch 16 at k = 11008 the one that reads activations from L2, batch
    16 on 768 tiles and more the one whose waves share an activation fragment among four tiles."""
    wt, wdq = _seeded(dtype, k, n, 1000 + k + n)
    # the device's dequantised values are the oracle's (bit-exact), on a corner of the matrix
    w_corner = np.array([[np.float32(0.02) * np.float32(orc.lib().orc_synth_normal(1000 + k + n, l * n + j))
                          for j in range(48)] for l in range(64)], dtype=np.float32)
    assert np.array_equal(oracle_roundtrip(orc, DT[dtype], w_corner), wdq[:64, :48].astype(np.float32))
    # ... and on 256 patches of 32 k (one quantisation block) x 16 outputs (one tile of rows) drawn
    # over the whole matrix, the last block of k, the last tile and the last column among them: a
    # packing or index error that only shows at large tile or group indices cannot hide behind the
    # device's own unpacking
    prng = np.random.default_rng(7 * k + n)
    lib = orc.lib()
    sd = 1000 + k + n
    corners = [(k // 32 - 1, (n - 1) // 16), (0, (n - 1) // 16), (k // 32 - 1, 0), (k // 128 * 4 - 1, n // 16 // 2)]
    picks = corners + [(int(prng.integers(0, k // 32)), int(prng.integers(0, (n + 15) // 16))) for _ in range(256 - len(corners))]
    for blk, tile in picks:
        l0, j0 = blk * 32, min(tile * 16, n - 16)
        patch = np.array([[np.float32(0.02) * np.float32(lib.orc_synth_normal(sd, (l0 + l) * n + j0 + j))
                           for j in range(16)] for l in range(32)], dtype=np.float32)
        assert np.array_equal(oracle_roundtrip(orc, DT[dtype], patch),
                              wdq[l0:l0 + 32, j0:j0 + 16].astype(np.float32)), (blk, tile)
    rng = np.random.default_rng(k + n)
    for batch in (1, 4, 8, 16):
        x = rng.standard_normal((batch, k)).astype(np.float32)
        res = rng.standard_normal((batch, n // 2 if gated else n)).astype(np.float32)
        pre = _f16(x) @ wdq
        if gated:
            g, u = pre[:, 0::2], pre[:, 1::2]
            want = g / (1 + np.exp(-g)) * u
            got = wt.gemv(dev(x), epilogue=_lib.EPI_SILU_GATE)
        else:
            want = pre + res
            got = wt.gemv(dev(x), residual=dev(res))
        assert rel_err(got, want) < 2e-5, (batch, rel_err(got, want))


def _norm64(h, kind, sc, bi, eps):
    h = h.astype(np.float64)
    if kind == _lib.NORM_RMSNORM:
        return sc * h / np.sqrt((h * h).mean(-1, keepdims=True) + np.float64(np.float32(eps)))
    mu = h.mean(-1, keepdims=True)
    return sc * (h - mu) / np.sqrt(((h - mu) ** 2).mean(-1, keepdims=True) + np.float64(np.float32(eps))) + bi


def _norm_gemv(wt, h, kind, sc, bi, eps, n_eff, epilogue=0, residual=None):
    lib = _lib.load()
    batch = h.shape[0]
    y = DeviceArray((batch, n_eff), np.float32)
    fused = C.c_int(-1)
    dh, dsc = dev(h), dev(sc)
    dbi = dev(bi) if bi is not None else None
    dres = dev(residual) if residual is not None else None
    _check(lib.coeus_op_norm_gemv(wt.h, dh.ptr, batch, kind, dsc.ptr, dbi.ptr if dbi else None, eps, None,
                                  dres.ptr if dres else None, epilogue, y.ptr, C.byref(fused), None))
    synchronize()
    return y.to_host(), fused.value


@pytest.mark.parametrize("dtype", ["q4_0", "q8_0"])
@pytest.mark.parametrize("k,n,gated,kind", [
    (4096, 12288, False, "rms"),   # q|k|v of the 7B shape
    (4096, 22016, True, "rms"),    # gate|up: two tiles per workgroup at batch 1
    (4096, 32000, False, "rms"),   # logits: two tiles per workgroup at batch 1
    (2048, 8192, False, "ln"),     # FFN-up of the 1B shape, LayerNorm
    (8192, 2048, False, "ln"),     # reduction length above 4096: eight statistics records per lane
    (8192, 2048, False, "rms"),
    (800, 520, False, "ln"),       # k = 32 (mod 128): the last group of blocks is a padded one
])
def test_norm_gemv_benchmark_shapes(orc, dtype, k, n, gated, kind):
    """coeus_op_norm_gemv: the norm folded into the decode matmul's staging (batch 1, 2 and 4: one,
    two and four pieces per lane where the width asks for it), and as its own launch for batch 8 and
    16, against a float64 norm -> f16 rounding -> float64 product on the oracle-dequantised
    weights.  The f32 norm arithmetic may round an activation to the neighbouring f16 value, so
    the bar is 1e-4 here (an indexing error is O(1))."""
    wt, wdq = _seeded(dtype, k, n, 2000 + k + n)
    rng = np.random.default_rng(3 * k + n)
    sc = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    bi = (0.1 * rng.standard_normal(k)).astype(np.float32) if kind == "ln" else None
    nk = _lib.NORM_LAYERNORM if kind == "ln" else _lib.NORM_RMSNORM
    n_eff = n // 2 if gated else n
    for batch in (1, 2, 4, 8, 16):
        h = (rng.standard_normal((batch, k)) * 1.5 + 0.3).astype(np.float32)
        res = rng.standard_normal((batch, n_eff)).astype(np.float32)
        xn = _f16(_norm64(h, nk, sc.astype(np.float64), None if bi is None else bi.astype(np.float64), 1e-5))
        pre = xn @ wdq
        if gated:
            g, u = pre[:, 0::2], pre[:, 1::2]
            want = g / (1 + np.exp(-g)) * u + res
            got, fused = _norm_gemv(wt, h, nk, sc, bi, 1e-5, n_eff, _lib.EPI_SILU_GATE, res)
        else:
            want = pre + res
            got, fused = _norm_gemv(wt, h, nk, sc, bi, 1e-5, n_eff, 0, res)
        # (folded for up to 4 rows whose f16 block fits 48 KiB, four rows only up to k = 4096)
        want_fused = batch <= 4 and k * batch <= 24576 and (batch <= 2 or k <= 4096)
        assert fused == (1 if want_fused else 0), (batch, fused)
        assert rel_err(got, want) < 1e-4, (batch, fused, rel_err(got, want))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("kind", ["ln", "rms"])
def test_norm_gemv_dense(orc, dtype, kind):
    """The same operator on f32 / bf16 weights (the 250M shapes): norm folded into the dense
    decode matmul's staging, products in f32."""
    k, n = 768, 2304
    rng = np.random.default_rng(9)
    w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    wt = Weight(DT[dtype], w)
    wdq = oracle_roundtrip(orc, DT[dtype], w).astype(np.float64)
    sc = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    bi = (0.1 * rng.standard_normal(k)).astype(np.float32) if kind == "ln" else None
    nk = _lib.NORM_LAYERNORM if kind == "ln" else _lib.NORM_RMSNORM
    for batch in (1, 3, 8, 16):
        h = (rng.standard_normal((batch, k)) * 1.5 + 0.3).astype(np.float32)
        want = _norm64(h, nk, sc.astype(np.float64), None if bi is None else bi.astype(np.float64), 1e-5) @ wdq
        got, fused = _norm_gemv(wt, h, nk, sc, bi, 1e-5, n)
        assert fused == 1 and rel_err(got, want) < 2e-5, (batch, rel_err(got, want))


# ------------------------------------------------------------------ decode attention, split context

def _to16(a, bf16, orc):
    """f32 array -> (uint16 storage bits, the float64 values they stand for)."""
    if bf16:
        r = orc.bf16_round(a)
        return (r.view(np.uint32) >> 16).astype(np.uint16), r.astype(np.float64)
    h = a.astype(np.float16)
    return h.view(np.uint16), h.astype(np.float64)


@pytest.mark.parametrize("hd,bf16", [(128, False), (128, True), (64, False), (64, True)])
@pytest.mark.parametrize("batch,heads,max_ctx", [(1, 4, 4096), (3, 5, 1024)])
def test_attention_decode_split_context(orc, hd, bf16, batch, heads, max_ctx):
    """coeus_op_attention_decode: one query per (sequence, head) against a 16-bit cache, the
    context split over 1 to 32 workgroups whose partial (max, sum, output) records are merged by
    the last split to finish, or by the separate merge kernel.  Against a float64 softmax
    attention over the first ctx cached positions (everything behind them holds large values that
    would show up if read), for contexts that leave most splits empty, end inside a split, inside a
    wave's tile of keys, and fill the cache.  Each call is repeated: the arrival counters must be
    back at zero after a launch."""
    lib = _lib.load()
    rng = np.random.default_rng(hd + batch * 7 + heads)
    inner = heads * hd
    qkv = rng.standard_normal((batch, 3 * inner)).astype(np.float32)
    K = rng.standard_normal((batch, heads, max_ctx, hd)).astype(np.float32)
    V = rng.standard_normal((batch, heads, max_ctx, hd)).astype(np.float32)
    kbits, k64 = _to16(K, bf16, orc)
    vbits, v64 = _to16(V, bf16, orc)
    dq, out = dev(qkv), DeviceArray((batch, inner), np.float32)
    kv = _lib.KV_BF16 if bf16 else _lib.KV_F16
    q64 = qkv[:, :inner].astype(np.float64).reshape(batch, heads, hd)
    for ctx in (1, 63, 300, max_ctx - 1, max_ctx):
        # poison what lies behind the context
        kb, vb = kbits.copy(), vbits.copy()
        poison = np.uint16(0x7BFF if not bf16 else 0x7F7F)  # largest finite f16 / bf16
        kb[:, :, ctx:, :] = poison
        vb[:, :, ctx:, :] = poison
        dk, dv = dev(kb), dev(vb)
        s = np.einsum("bhd,bhcd->bhc", q64, k64[:, :, :ctx]) / np.sqrt(hd)
        p = np.exp(s - s.max(-1, keepdims=True))
        want = np.einsum("bhc,bhcd->bhd", p / p.sum(-1, keepdims=True), v64[:, :, :ctx]).reshape(batch, inner)
        results = {}
        for nsplit in (0, 1, 2, 8, 16, 32):
            for merge in (_lib.MERGE_IN_KERNEL, _lib.MERGE_SEPARATE):
                for rep in range(2):
                    out.zero_()
                    _check(lib.coeus_op_attention_decode(dq.ptr, dk.ptr, dv.ptr, kv, batch, heads, hd, max_ctx,
                                                         ctx, nsplit, merge, out.ptr, None))
                    got = out.to_host()
                    err = rel_err(got, want)
                    assert err < 1e-5, (ctx, nsplit, merge, rep, err)
                results[(nsplit, merge)] = got
            # the two merges add the same records in the same order
            assert rel_err(results[(nsplit, 0)], results[(nsplit, 1)]) < 2e-6, (ctx, nsplit)
        dk.free()
        dv.free()


@pytest.mark.parametrize("hd,bf16", [(128, False), (128, True), (64, False), (64, True)])
def test_attention_decode_large_cache(orc, hd, bf16):
    """A cache of more than 100 MB, as a batch of 13 sequences: the same float64 check, for a
    context inside a wave's tile of keys and a full one, with the library's split count (one
    workgroup per sequence and head at this batch) and with two splits."""
    lib = _lib.load()
    batch, heads, max_ctx = 13, 1024 // hd, 2048          # 13 * 1024 * 2048 * 4 bytes = 109 MB
    rng = np.random.default_rng(hd + 1000)
    inner = heads * hd
    qkv = rng.standard_normal((batch, 3 * inner)).astype(np.float32)
    K = rng.standard_normal((batch, heads, max_ctx, hd)).astype(np.float32)
    V = rng.standard_normal((batch, heads, max_ctx, hd)).astype(np.float32)
    kbits, k64 = _to16(K, bf16, orc)
    vbits, v64 = _to16(V, bf16, orc)
    dq, dk, dv, out = dev(qkv), dev(kbits), dev(vbits), DeviceArray((batch, inner), np.float32)
    kv = _lib.KV_BF16 if bf16 else _lib.KV_F16
    q64 = qkv[:, :inner].astype(np.float64).reshape(batch, heads, hd)
    for ctx in (300, max_ctx):
        s = np.einsum("bhd,bhcd->bhc", q64, k64[:, :, :ctx]) / np.sqrt(hd)
        p = np.exp(s - s.max(-1, keepdims=True))
        want = np.einsum("bhc,bhcd->bhd", p / p.sum(-1, keepdims=True), v64[:, :, :ctx]).reshape(batch, inner)
        for nsplit in (0, 2):
            out.zero_()
            _check(lib.coeus_op_attention_decode(dq.ptr, dk.ptr, dv.ptr, kv, batch, heads, hd, max_ctx, ctx,
                                                 nsplit, _lib.MERGE_IN_KERNEL, out.ptr, None))
            err = rel_err(out.to_host(), want)
            assert err < 1e-5, (ctx, nsplit, err)


def test_attention_decode_argument_errors():
    lib = _lib.load()
    from coeus_amd.plugin import ProcessingError
    d = DeviceArray((4096,), np.float32)
    for args in [(_lib.KV_F32, 1, 2, 64, 16, 4, 0, 0), (_lib.KV_F16, 1, 2, 48, 16, 4, 0, 0),
                 (_lib.KV_F16, 1, 2, 64, 16, 17, 0, 0), (_lib.KV_F16, 1, 2, 64, 16, 0, 0, 0),
                 (_lib.KV_F16, 1, 2, 64, 16, 4, 33, 0), (_lib.KV_F16, 1, 2, 64, 16, 4, 0, 2),
                 (_lib.KV_F16, 0, 2, 64, 16, 4, 0, 0)]:
        kvd, b, h, hd, mc, ctx, ns, mg = args
        with pytest.raises(ProcessingError):
            _check(lib.coeus_op_attention_decode(d.ptr, d.ptr, d.ptr, kvd, b, h, hd, mc, ctx, ns, mg, d.ptr, None))
