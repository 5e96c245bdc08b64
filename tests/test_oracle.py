"""Pins the CPU oracle (oracle/coeus_oracle.c) before anything is compared with it.

The reference (rustllm-core/plugins/model-transformer/src/lib.rs = MT,
rustllm-core/src/core/model.rs = CM) holds no golden vectors for this path (its tests check
lengths and loose invariants, MT:1123-1224), so each oracle function is pinned by: the
reference's own test assertions restated, closed forms, brute force on integer inputs, library
routines it must reduce to, and an independent float64 implementation (tests/f64_model.py).
"""
import ctypes as C
import math

import numpy as np
import pytest

import f64_model


# ------------------------------------------------------------------ config (CM:776-807)

def test_config_defaults_and_validate(orc):
    c = orc.default_config()
    assert (c.hidden_dim, c.num_layers, c.num_heads) == (768, 12, 12)
    assert (c.intermediate_dim, c.vocab_size, c.max_seq_len) == (3072, 50257, 1024)
    assert c.dropout == np.float32(0.1) and c.attention_dropout == np.float32(0.1)
    assert c.layer_norm_eps == np.float32(1e-5)
    assert c.use_bias == 1
    assert orc.validate(c) == (0, None)
    # the four invalid cases of CM:792-806
    assert orc.validate(orc.default_config(hidden_dim=767)) == (2, "hidden_dim")
    assert orc.validate(orc.default_config(num_layers=0)) == (2, "num_layers")
    assert orc.validate(orc.default_config(vocab_size=0)) == (2, "vocab_size")
    assert orc.validate(orc.default_config(max_seq_len=0)) == (2, "max_seq_len")
    assert orc.validate(orc.default_config(hidden_dim=0)) == (2, "hidden_dim")


# ------------------------------------------------------------------ parameters

def test_param_count_and_layout_closed_form(orc):
    c = orc.default_config()
    n = orc.num_parameters(c)
    assert 160_000_000 < n < 170_000_000  # MT:1143-1144
    # MT:541-580 evaluated by hand for the default config
    H, L, I, V, S = 768, 12, 3072, 50257, 1024
    per_layer = 4 * H * H + 4 * H + 2 * H + 2 * H * I + I + H + 2 * H
    assert n == V * H + S * H + L * per_layer + 2 * H + H * V + V == 163_087_441
    lay = orc.layout(c)
    assert lay.first_layer_offset == 38_597_376 and lay.layer_stride == 7_087_872
    assert (lay.ln1_scale, lay.ln1_bias, lay.wq, lay.wk, lay.wv, lay.wo) == (
        0, 768, 1536, 1536 + 589_824, 1536 + 2 * 589_824, 1536 + 3 * 589_824)
    assert (lay.bq, lay.ln2_scale, lay.ln2_bias) == (2_360_832, 2_363_904, 2_364_672)
    assert (lay.w_up, lay.w_down, lay.b_up, lay.b_down) == (
        2_365_440, 4_724_736, 7_084_032, 7_087_104)
    assert lay.final_ln_offset == 123_651_840 and lay.output_proj_offset == 123_653_376
    assert lay.used_params == 162_250_752 and n - lay.used_params == 836_689
    # independent derivation agrees for a biasless, gated, decoupled-head config
    c2 = orc.default_config(hidden_dim=64, num_layers=3, num_heads=4, head_dim=8,
                            intermediate_dim=96, vocab_size=100, max_seq_len=16, use_bias=0,
                            activation=1)
    first, stride, rel = f64_model.offsets(c2)
    l2 = orc.layout(c2)
    assert (l2.first_layer_offset, l2.layer_stride) == (first, stride)
    for name, field in [("wq", "wq"), ("wo", "wo"), ("w_gate", "w_gate"), ("w_up", "w_up"),
                        ("w_down", "w_down"), ("ln2_s", "ln2_scale")]:
        assert getattr(l2, field) == rel[name][0]


def test_default_init_closed_form(orc):
    p = orc.init_default(100_000, 768)
    assert p[0] == 0.0
    i = np.arange(100_000, dtype=np.float32)
    want = np.sin((i * np.float32(0.1234567)).astype(np.float64)) * math.sqrt(2.0 / 768)
    assert np.abs(p - want).max() < 2e-7
    # clamp bound is active when sqrt(2/hidden) > 0.1
    p4 = orc.init_default(5000, 4)
    assert p4.max() == np.float32(0.1) and p4.min() == np.float32(-0.1)
    # index is converted to f32 before the multiply (rounds above 2^24)
    big = orc.init_default((1 << 24) + 4, 768)
    f = np.float32((1 << 24) + 3)  # rounds to 2^24+4
    want_big = math.sin(float(f * np.float32(0.1234567))) * math.sqrt(2.0 / 768)
    assert abs(big[(1 << 24) + 3] - want_big) < 2e-7


# ------------------------------------------------------------------ math

def test_matmul_integer_brute_force_exact(orc):
    rng = np.random.default_rng(1)
    for (m, n, k) in [(1, 1, 1), (3, 5, 7), (65, 70, 130), (2, 129, 64)]:
        a = rng.integers(-8, 9, size=(m, k)).astype(np.float32)
        b = rng.integers(-8, 9, size=(k, n)).astype(np.float32)
        want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
        assert np.array_equal(orc.matmul(a, b, ref=True), want)
        assert np.array_equal(orc.matmul(a, b, ref=False), want)


def test_matmul_is_ascending_k_dot_without_fma(orc):
    rng = np.random.default_rng(2)
    m, n, k = 5, 67, 131  # block edges that are not multiples of 64
    a = rng.standard_normal((m, k)).astype(np.float32)
    b = rng.standard_normal((k, n)).astype(np.float32)
    want = np.zeros((m, n), dtype=np.float32)
    for l in range(k):  # one rounded product and one rounded add per step
        want = want + (a[:, l:l + 1] * b[l:l + 1, :]).astype(np.float32)
    got_ref = orc.matmul(a, b, ref=True)
    got_fast = orc.matmul(a, b, ref=False)
    assert np.array_equal(got_ref.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(got_fast.view(np.uint32), want.view(np.uint32))
    # a transposed operand or a wrong index would miss the float64 product by O(1)
    assert np.abs(got_ref - a.astype(np.float64) @ b.astype(np.float64)).max() < 1e-4


def test_softmax(orc):
    out = orc.softmax([1.0, 2.0, 3.0])
    assert abs(out.sum() - 1.0) < 1e-6 and (out > 0).all()  # MT:1178-1192
    assert out[2] > out[1] > out[0]
    assert np.allclose(out, [0.09003057, 0.24472847, 0.66524096], atol=1e-7)
    masked = orc.softmax([0.5, -np.inf, 0.25, -np.inf])
    assert masked[1] == 0.0 and masked[3] == 0.0 and abs(masked.sum() - 1) < 1e-6
    big = orc.softmax([1000.0, 1001.0])  # max-subtraction keeps it finite
    assert np.allclose(big, [0.26894143, 0.7310586], atol=1e-7)


def test_gelu(orc):
    assert abs(orc.gelu(0.0)) < 1e-6 and orc.gelu(1.0) > 0.8 and orc.gelu(-1.0) < -0.1  # MT:1170
    assert abs(orc.gelu(1.0) - 0.8411920) < 1e-6
    assert abs(orc.gelu(-1.0) + 0.1588080) < 1e-6
    for x in (-3.0, -0.5, 0.3, 2.5):
        want = 0.5 * x * (1 + math.tanh(math.sqrt(2 / math.pi) * (x + 0.044715 * x ** 3)))
        assert abs(orc.gelu(x) - want) < 1e-6


def test_layer_norm(orc):
    out = orc.layer_norm([1, 2, 3, 4], [1] * 4, [0] * 4, 1e-5)
    mean = out.mean()
    assert abs(mean) < 0.01 and abs(((out - mean) ** 2).mean() - 1) < 0.01  # MT:1153-1167
    want = (np.array([1, 2, 3, 4.0]) - 2.5) / math.sqrt(1.25 + 1e-5)
    assert np.abs(out - want).max() < 1e-6
    # statistics span the whole slice; scale/bias are indexed i % len (MT:124)
    import torch
    rng = np.random.default_rng(3)
    S, H = 7, 24
    x = rng.standard_normal(S * H).astype(np.float32) * 3 + 1
    sc = rng.standard_normal(H).astype(np.float32)
    bi = rng.standard_normal(H).astype(np.float32)
    got = orc.layer_norm(x, sc, bi, 1e-5)
    tx = torch.from_numpy(x).double()
    want = torch.nn.functional.layer_norm(
        tx, (S * H,), torch.from_numpy(np.tile(sc, S)).double(),
        torch.from_numpy(np.tile(bi, S)).double(), 1e-5).numpy()
    assert np.abs(got - want).max() < 2e-6
    # and it is NOT the per-token statistic
    per_tok = torch.nn.functional.layer_norm(
        tx.reshape(S, H), (H,), torch.from_numpy(sc).double(), torch.from_numpy(bi).double(),
        1e-5).numpy().ravel()
    assert np.abs(got - per_tok).max() > 1e-2
    # one row reduces to the standard LayerNorm
    got1 = orc.layer_norm(x[:H], sc, bi, 1e-5)
    assert np.abs(got1 - per_tok[:H]).max() < 2e-6


def test_positional_encoding(orc):
    t = orc.positional_encoding(10, 8)
    assert t[:5].size == 40 and not np.array_equal(t[0], t[1])  # MT:1195-1206
    assert np.array_equal(t[0], np.array([0, 1] * 4, dtype=np.float32))
    ang = np.array([1.0, 0.1, 0.01, 0.001])
    assert np.abs(t[1, 0::2] - np.sin(ang)).max() < 1e-6
    assert np.abs(t[1, 1::2] - np.cos(ang)).max() < 1e-6
    big = orc.positional_encoding(64, 48)
    assert np.abs(big - f64_model.pe_table(64, 48)).max() < 5e-6
    # odd hidden_dim leaves the last column zero (i runs to hidden/2, MT:402)
    odd = orc.positional_encoding(4, 5)
    assert np.array_equal(odd[:, 4], np.zeros(4, dtype=np.float32))


def test_causal_mask(orc):
    assert np.array_equal(orc.causal_mask(5), np.tril(np.ones((5, 5), dtype=np.float32)))


# ------------------------------------------------------------------ attention / ffn / block

def _mha_f64(x, w, b, heads, causal):
    S, H = x.shape
    d = H // heads
    wq, wk, wv, wo = (w[i * H * H:(i + 1) * H * H].reshape(H, H) for i in range(4))
    q, k, v = x @ wq, x @ wk, x @ wv
    if b is not None:
        q, k, v = q + b[:H], k + b[H:2 * H], v + b[2 * H:3 * H]
    out = np.zeros((S, H))
    for h in range(heads):
        sl = slice(h * d, (h + 1) * d)
        sc = q[:, sl] @ k[:, sl].T / math.sqrt(d)
        if causal:
            sc = np.where(np.tril(np.ones((S, S), dtype=bool)), sc, -np.inf)
        pr = np.exp(sc - sc.max(-1, keepdims=True))
        pr /= pr.sum(-1, keepdims=True)
        out[:, sl] = pr @ v[:, sl]
    out = out @ wo
    return out + b[3 * H:] if b is not None else out


def test_mha_reference_test_inputs_closed_form(orc):
    # the inputs of MT:1209-1219; the reference asserts only the length, the value is derived:
    # V-proj = 8*0.1*0.01 = 0.008 everywhere, softmax uniform, O-proj = 8*0.008*0.01
    S, H = 3, 8
    out = orc.mha_forward(H, 2, np.full(S * H, 1.0), np.full(S * H, 0.5), np.full(S * H, 0.1),
                          np.full(4 * H * H, 0.01), None, None, S)
    assert out.size == S * H
    assert np.abs(out - 6.4e-4).max() < 1e-9


def test_mha_against_float64(orc):
    rng = np.random.default_rng(4)
    S, H, heads = 9, 32, 4
    x = rng.standard_normal((S, H)).astype(np.float32)
    w = (rng.standard_normal(4 * H * H) * 0.2).astype(np.float32)
    b = (rng.standard_normal(4 * H) * 0.1).astype(np.float32)
    mask = orc.causal_mask(S)
    got = orc.mha_forward(H, heads, x, x, x, w, b, mask, S).reshape(S, H)
    want = _mha_f64(x.astype(np.float64), w.astype(np.float64), b.astype(np.float64), heads, True)
    assert np.abs(got - want).max() < 2e-5
    # causal row 0 attends only to itself: equals (V[0]) . Wo + bo
    wv = w[2 * H * H:3 * H * H].reshape(H, H).astype(np.float64)
    wo = w[3 * H * H:].reshape(H, H).astype(np.float64)
    row0 = (x[0].astype(np.float64) @ wv + b[2 * H:3 * H]) @ wo + b[3 * H:]
    assert np.abs(got[0] - row0).max() < 2e-5
    # without a mask row 0 sees every key, so the result must differ
    nomask = orc.mha_forward(H, heads, x, x, x, w, b, None, S).reshape(S, H)
    assert np.abs(nomask[0] - got[0]).max() > 1e-3
    want_nm = _mha_f64(x.astype(np.float64), w.astype(np.float64), b.astype(np.float64), heads, False)
    assert np.abs(nomask - want_nm).max() < 2e-5


def test_ffn_against_float64(orc):
    rng = np.random.default_rng(5)
    S, H, I = 5, 16, 40
    x = rng.standard_normal((S, H)).astype(np.float32)
    w = (rng.standard_normal(2 * H * I) * 0.3).astype(np.float32)
    b = (rng.standard_normal(I + H) * 0.1).astype(np.float32)
    got = orc.ffn_forward(H, I, x, w, b, S).reshape(S, H)
    up = x.astype(np.float64) @ w[:H * I].reshape(H, I) + b[:I]
    want = f64_model.gelu(up) @ w[H * I:].reshape(I, H).astype(np.float64) + b[I:]
    assert np.abs(got - want).max() < 2e-5
    nb = orc.ffn_forward(H, I, x, w, None, S).reshape(S, H)
    want_nb = f64_model.gelu(x.astype(np.float64) @ w[:H * I].reshape(H, I)) @ w[H * I:].reshape(I, H)
    assert np.abs(nb - want_nb).max() < 2e-5


# ------------------------------------------------------------------ whole forward

def _small(orc, **over):
    kw = dict(hidden_dim=48, num_layers=3, num_heads=4, intermediate_dim=80, vocab_size=211,
              max_seq_len=32)
    kw.update(over)
    return orc.default_config(**kw)


def _rel_err(got, want):
    return np.abs(got - want).max() / np.abs(want).max()


@pytest.mark.parametrize("use_bias", [1, 0])
def test_forward_reference_mode_against_float64(orc, use_bias):
    cfg = _small(orc, use_bias=use_bias)
    params = orc.init_seeded(cfg, 11)
    ids = orc.synth_ids(12, cfg.vocab_size, 19)
    rc, last, allr = orc.forward(cfg, params, ids, all_rows=True, fast=False)
    assert rc == 0
    want = f64_model.forward_all(cfg, params, ids)
    assert _rel_err(allr, want) < 2e-5
    assert np.array_equal(last, allr[-1])
    assert np.array_equal(allr.argmax(-1), want.argmax(-1))
    # the reference's own sin init (MT:604-611) through the same comparison
    p_sin = orc.init_default(orc.num_parameters(cfg), cfg.hidden_dim)
    rc, last = orc.forward(cfg, p_sin, ids, fast=False)
    want_sin = f64_model.forward_all(cfg, p_sin, ids)[-1]
    assert rc == 0 and _rel_err(last, want_sin) < 2e-5


def test_forward_paths_agree_bitwise(orc):
    """Literal matmul vs reordered matmul, literal forward vs generalised forward."""
    cfg = _small(orc)
    params = orc.init_seeded(cfg, 21)
    ids = orc.synth_ids(22, cfg.vocab_size, 13)
    _, a = orc.forward(cfg, params, ids, fast=False)
    _, b = orc.forward(cfg, params, ids, fast=True)
    _, c = orc.forward(cfg, params, ids, fast=True, force_general=True)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert np.array_equal(a.view(np.uint32), c.view(np.uint32))


def test_forward_matches_reference_unit_test_shape(orc):
    """MT:1137-1150: three ids in, vocab-size logits out; seq_len 1 equals per-token norm."""
    cfg = _small(orc)
    params = orc.init_default(orc.num_parameters(cfg), cfg.hidden_dim)
    rc, out = orc.forward(cfg, params, [100, 200, 30])
    assert rc == 0 and out.shape == (cfg.vocab_size,)
    rc1, one = orc.forward(cfg, params, [7])
    cfg_tok = _small(orc, norm_scope=1)
    rc2, one_tok = orc.forward(cfg_tok, params, [7])
    assert rc1 == 0 and rc2 == 0 and np.array_equal(one.view(np.uint32), one_tok.view(np.uint32))


def test_forward_errors(orc):
    cfg = _small(orc)
    params = orc.init_seeded(cfg, 1)
    assert orc.forward(cfg, params, [cfg.vocab_size])[0] == 1          # MT:816-822
    assert orc.forward(cfg, params, list(range(33)))[0] == 1           # MT:797-802
    assert orc.forward(cfg, params, [])[0] == 1                        # reference panics (MT:915)
    assert orc.forward(cfg, params[:1000], [1, 2])[0] == 1             # MT:661-669
    assert orc.forward(_small(orc, hidden_dim=50), params, [1])[0] == 2


@pytest.mark.parametrize("over", [
    dict(norm_scope=1),
    dict(norm_scope=1, norm=1, activation=1, use_bias=0),
    dict(norm_scope=1, head_dim=8),               # inner width 32 != hidden 48
    dict(norm=1),                                  # whole-slice RMS
])
def test_forward_extensions_against_float64(orc, over):
    cfg = _small(orc, **over)
    params = orc.init_seeded(cfg, 31)
    ids = orc.synth_ids(32, cfg.vocab_size, 17)
    rc, last, allr = orc.forward(cfg, params, ids, all_rows=True)
    assert rc == 0
    want = f64_model.forward_all(cfg, params, ids)
    assert _rel_err(allr, want) < 2e-5


def test_per_token_scope_is_causal_and_whole_slice_is_not(orc):
    cfg_tok = _small(orc, norm_scope=1)
    cfg_seq = _small(orc)
    params = orc.init_seeded(cfg_tok, 41)
    ids = orc.synth_ids(42, cfg_tok.vocab_size, 12)
    _, _, full_tok = orc.forward(cfg_tok, params, ids, all_rows=True)
    _, _, pre_tok = orc.forward(cfg_tok, params, ids[:7], all_rows=True)
    assert np.array_equal(full_tok[:7].view(np.uint32), pre_tok.view(np.uint32))
    _, _, full_seq = orc.forward(cfg_seq, params, ids, all_rows=True)
    _, _, pre_seq = orc.forward(cfg_seq, params, ids[:7], all_rows=True)
    assert not np.array_equal(full_seq[:7], pre_seq)


# ------------------------------------------------------------------ KV-cache session

@pytest.mark.parametrize("over", [dict(), dict(norm=1, activation=1, use_bias=0, head_dim=8),
                                  dict(kv_dtype=1), dict(kv_dtype=2)])
def test_session_incremental_equals_full_recompute(orc, over):
    cfg = _small(orc, norm_scope=1, **over)
    params = orc.init_seeded(cfg, 51)
    ids = orc.synth_ids(52, cfg.vocab_size, 14)
    _, _, full = orc.forward(cfg, params, ids, all_rows=True)
    s = orc.Session(cfg, params, 32)
    rc, last, pre = s.feed(ids[:9], all_rows=True)
    assert rc == 0 and s.position == 9
    assert np.array_equal(pre.view(np.uint32), full[:9].view(np.uint32))
    for i in range(9, 14):
        rc, step = s.feed(ids[i:i + 1])
        assert rc == 0
        assert np.array_equal(step.view(np.uint32), full[i].view(np.uint32)), i
    assert s.feed(np.concatenate([ids, ids]))[0] == 1  # 14 + 28 would exceed max_ctx = 32
    s.reset()
    rc, again = s.feed(ids[:9])
    assert np.array_equal(again.view(np.uint32), full[8].view(np.uint32))
    s.close()


# ------------------------------------------------------------------ number formats

def test_f16_conversions_against_numpy(orc):
    L = orc.lib()
    allh = np.arange(65536, dtype=np.uint16)
    want = allh.view(np.float16).astype(np.float32)
    got = np.array([L.orc_f16_to_f32(int(h)) for h in allh], dtype=np.float32)
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))
    assert np.isnan(got[~ok]).all()
    rng = np.random.default_rng(6)
    xs = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 5.96e-8, 2.98e-8, 2.9802323e-8,
                  6.1e-5, 6.097e-5, np.inf, -np.inf], dtype=np.float32),
        # exact ties between neighbouring halfs
        (allh[:31743:7].view(np.float16).astype(np.float64) +
         allh[1:31744:7].view(np.float16).astype(np.float64)).astype(np.float32) / 2,
    ])
    with np.errstate(over="ignore"):
        want16 = xs.astype(np.float16).view(np.uint16)
    got16 = np.array([L.orc_f32_to_f16(float(x)) for x in xs], dtype=np.uint16)
    assert np.array_equal(got16, want16)


def test_bf16_round_against_torch(orc):
    import torch
    rng = np.random.default_rng(7)
    x = (rng.standard_normal(50000) * 10.0 ** rng.integers(-20, 20, 50000)).astype(np.float32)
    want = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
    L = orc.lib()
    got = np.array([L.orc_bf16_round(float(v)) for v in x[:5000]], dtype=np.float32)
    assert np.array_equal(got, want[:5000])
    assert np.array_equal(orc.bf16_round(x), want)


def _np_q8_0(x):
    xb = x.reshape(-1, 32).astype(np.float32)
    d = (np.abs(xb).max(1) / np.float32(127.0)).astype(np.float32)
    idv = np.where(d != 0, np.float32(1.0) / np.where(d != 0, d, 1), 0).astype(np.float32)
    v = (xb * idv[:, None]).astype(np.float32)
    q = (np.sign(v) * np.floor(np.abs(v) + np.float32(0.5))).astype(np.int8)  # roundf: half away
    return q.ravel(), d.astype(np.float16).view(np.uint16)


def _np_q4_0(x):
    xb = x.reshape(-1, 32).astype(np.float32)
    idx = np.abs(xb).argmax(1)  # first index of the largest magnitude, as the strict '<' scan
    mx = xb[np.arange(len(xb)), idx]
    d = (mx / np.float32(-8.0)).astype(np.float32)
    idv = np.where(d != 0, np.float32(1.0) / np.where(d != 0, d, 1), 0).astype(np.float32)
    v = (xb * idv[:, None]).astype(np.float32) + np.float32(8.5)
    q = np.minimum(15, v.astype(np.int32)).astype(np.uint8)
    packed = q[:, :16] | (q[:, 16:] << 4)
    return packed.ravel(), d.astype(np.float16).view(np.uint16)


def test_q8_0_convention(orc):
    rng = np.random.default_rng(8)
    x = (rng.standard_normal(32 * 200) * 0.02).astype(np.float32)
    x[64:96] = 0  # an all-zero block
    qs, ds = orc.quantize_q8_0(x)
    wq, wd = _np_q8_0(x)
    assert np.array_equal(qs, wq) and np.array_equal(ds, wd)
    deq = orc.dequantize_q8_0(qs, ds)
    assert np.array_equal(deq, (wq.astype(np.float32).reshape(-1, 32) *
                                wd.view(np.float16).astype(np.float32)[:, None]).ravel())
    amax = np.abs(x.reshape(-1, 32)).max(1)
    # half a step of rounding plus the f16 rounding of the scale
    assert (np.abs(deq - x).reshape(-1, 32).max(1) <= amax / 127 * 0.5 + amax * 2.0 ** -11 + 1e-12).all()
    assert (deq[64:96] == 0).all()


def test_q4_0_convention(orc):
    rng = np.random.default_rng(9)
    x = (rng.standard_normal(32 * 200) * 0.02).astype(np.float32)
    x[32:64] = 0
    qs, ds = orc.quantize_q4_0(x)
    wq, wd = _np_q4_0(x)
    assert np.array_equal(qs, wq) and np.array_equal(ds, wd)
    deq = orc.dequantize_q4_0(qs, ds)
    d32 = wd.view(np.float16).astype(np.float32)
    lo = (wq.reshape(-1, 16) & 15).astype(np.int32) - 8
    hi = (wq.reshape(-1, 16) >> 4).astype(np.int32) - 8
    want = np.concatenate([lo, hi], axis=1).astype(np.float32) * d32[:, None]
    assert np.array_equal(deq, want.ravel())
    # the largest-magnitude element maps to q=0 (value -8*d) and is reproduced up to f16 rounding of d
    xb = x.reshape(-1, 32)
    idx = np.abs(xb).argmax(1)
    mx = xb[np.arange(len(xb)), idx]
    got_mx = deq.reshape(-1, 32)[np.arange(len(xb)), idx]
    assert (np.abs(got_mx - mx) <= np.abs(mx) * 2.0 ** -10).all()
    step = np.abs(mx) / 8
    assert (np.abs(deq - x).reshape(-1, 32).max(1) <= step * 1.001 + 1e-12).all()


def test_apply_weight_dtype_touches_only_linear_weights(orc):
    for wd in (1, 2, 3):
        cfg = _small(orc, hidden_dim=64, intermediate_dim=96, norm_scope=1, weight_dtype=wd)
        params = orc.init_seeded(cfg, 61)
        q = orc.apply_weight_dtype(cfg, params)
        lay = orc.layout(cfg)
        base = lay.first_layer_offset
        # norm parameters and biases untouched
        for off, n in [(lay.ln1_scale, 64), (lay.bq, 64), (lay.b_up, 96), (lay.ln2_bias, 64)]:
            assert np.array_equal(q[base + off: base + off + n], params[base + off: base + off + n])
        assert np.array_equal(q[lay.final_ln_offset:lay.output_proj_offset],
                              params[lay.final_ln_offset:lay.output_proj_offset])
        wq0 = params[base + lay.wq: base + lay.wq + 64 * 64].reshape(64, 64)
        got = q[base + lay.wq: base + lay.wq + 64 * 64].reshape(64, 64)
        if wd == 1:
            want = orc.bf16_round(wq0)
            assert np.array_equal(q[:lay.token_embed_size], orc.bf16_round(params[:lay.token_embed_size]))
        else:
            quant, deq = ((orc.quantize_q8_0, orc.dequantize_q8_0) if wd == 2 else
                          (orc.quantize_q4_0, orc.dequantize_q4_0))
            # blocks run along the input dimension (rows of the [in, out] matrix) per output column
            want = np.stack([deq(*quant(wq0[:, j].copy())) for j in range(64)], axis=1)
            assert np.array_equal(q[:lay.token_embed_size], params[:lay.token_embed_size])
        assert np.array_equal(got, want)


# ------------------------------------------------------------------ synthetic data

def test_seeded_generator(orc):
    cfg = _small(orc)
    a = orc.init_seeded(cfg, 5)
    b = orc.init_seeded(cfg, 5)
    c = orc.init_seeded(cfg, 6)
    assert np.array_equal(a, b) and not np.array_equal(a, c)
    lay = orc.layout(cfg)
    emb = a[:lay.token_embed_size]
    assert abs(emb.mean()) < 5e-4 and abs(emb.std() - 0.02) < 5e-4
    base = lay.first_layer_offset
    s1 = a[base + lay.ln1_scale: base + lay.ln1_scale + cfg.hidden_dim]
    assert abs(s1.mean() - 1.0) < 0.02
    fin = a[lay.final_ln_offset: lay.final_ln_offset + cfg.hidden_dim]
    assert abs(fin.mean() - 1.0) < 0.02
    finb = a[lay.final_ln_offset + cfg.hidden_dim: lay.output_proj_offset]
    assert abs(finb.mean()) < 0.02
    z = np.array([orc.lib().orc_synth_normal(9, i) for i in range(20000)])
    assert abs(z.mean()) < 0.03 and abs(z.std() - 1.0) < 0.03 and np.abs(z).max() < 4.9
    ids = orc.synth_ids(3, 211, 5000)
    assert ids.max() < 211 and len(np.unique(ids)) > 200


# ------------------------------------------------------------------ quantiser known answers
# Blocks worked out by hand from the published GGML reference quantisers (quantize_row_q4_0_ref /
# quantize_row_q8_0_ref), with values that make every intermediate exact in f32, so a wrong
# rounding offset, clamp, tie rule, nibble order or scale sign changes a literal byte below.

def test_q4_0_known_answer_blocks(orc):
    a = np.zeros(32, dtype=np.float32)
    # largest magnitude 8 appears twice: the first (-8.0) wins, so d = -8 / -8 = 1 and x/d = x
    a[:10] = [-8.0, 8.0, 0.5, 0.49, -0.5, -0.51, 7.49, 7.5, -7.5, -7.51]
    a[16] = 3.0
    # trunc(x + 8.5): -8 -> 0; 8 -> 16 -> clamped 15; 0.5 -> 9; 0.49 -> 8; -0.5 -> 8; -0.51 -> 7;
    # 7.49 -> 15; 7.5 -> 16 -> 15; -7.5 -> 1; -7.51 -> 0; zeros -> 8; element 16 (3.0 -> 11) is the
    # high nibble of byte 0
    want_a = bytes([0xB0, 0x8F, 0x89, 0x88, 0x88, 0x87, 0x8F, 0x8F, 0x81, 0x80] + [0x88] * 6)
    b = np.zeros(32, dtype=np.float32)
    # positive maximum 4.0 at index 5: d = 4 / -8 = -0.5, x/d = -2x
    b[:6] = [-3.75, 1.0, 0.25, 0.26, 0.0, 4.0]
    # -3.75 -> 7.5 + 8.5 = 16 -> 15; 1.0 -> 6.5 -> 6; 0.25 -> 8.0 -> 8; 0.26 -> 7.98 -> 7; 4.0 -> 0.5 -> 0
    want_b = bytes([0x8F, 0x86, 0x88, 0x87, 0x88, 0x80] + [0x88] * 10)
    z = np.zeros(32, dtype=np.float32)  # d = 0 / -8 = -0.0, id = 0, every q = trunc(8.5) = 8
    qs, ds = orc.quantize_q4_0(np.concatenate([a, b, z]))
    assert bytes(qs[:16]) == want_a and bytes(qs[16:32]) == want_b and bytes(qs[32:]) == bytes([0x88] * 16)
    assert list(ds) == [0x3C00, 0xB800, 0x8000]  # f16 1.0, -0.5, -0.0 (the sign of the zero scale is kept)
    deq = orc.dequantize_q4_0(qs, ds)
    want_deq_a = np.zeros(32, dtype=np.float32)
    want_deq_a[:10] = [-8, 7, 1, 0, 0, -1, 7, 7, -7, -8]
    want_deq_a[16] = 3
    want_deq_b = np.zeros(32, dtype=np.float32)
    want_deq_b[:6] = [-3.5, 1.0, 0.0, 0.5, 0.0, 4.0]
    assert np.array_equal(deq[:32], want_deq_a) and np.array_equal(deq[32:64], want_deq_b)
    assert np.array_equal(deq[64:], np.zeros(32, dtype=np.float32))


def test_q8_0_known_answer_blocks(orc):
    a = np.zeros(32, dtype=np.float32)
    # amax = 127: d = 1, q = roundf(x) (halves away from zero)
    a[:12] = [127.0, -127.0, 0.5, -0.5, 1.5, -1.5, 2.4999, 0.49999, 63.5, -63.5, 2.5, -2.5]
    want_a = [127, -127, 1, -1, 2, -2, 2, 0, 64, -64, 3, -3] + [0] * 20
    b = np.zeros(32, dtype=np.float32)
    # amax = 63.5: d = 0.5, x/d = 2x
    b[:6] = [63.5, 0.25, -0.25, 0.75, -0.74, 0.24]
    want_b = [127, 1, -1, 2, -1, 0] + [0] * 26
    z = np.zeros(32, dtype=np.float32)
    qs, ds = orc.quantize_q8_0(np.concatenate([a, b, z]))
    assert list(qs[:32]) == want_a and list(qs[32:64]) == want_b and not qs[64:].any()
    assert list(ds) == [0x3C00, 0x3800, 0x0000]
    deq = orc.dequantize_q8_0(qs, ds)
    assert np.array_equal(deq[:32], np.array(want_a, dtype=np.float32))
    assert np.array_equal(deq[32:64], np.array(want_b, dtype=np.float32) * np.float32(0.5))
