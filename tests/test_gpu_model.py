"""GPU parity of the whole forward pass, through the plugin surface
(TransformerModelPlugin -> create_builder() -> build(config) -> model.forward(ids)), against the
CPU oracle on identical parameters and token ids.

Bars (from the task statement): argmax token ids identical; logits within max-abs relative 1e-3
on the f32 path and 2e-2 on the bf16 / quantised paths."""
import numpy as np
import pytest

from coeus_amd import (ConfigError, ProcessingError, Transformer250MConfig, TransformerModelBuilder,
                       TransformerModelPlugin)
from gpu_util import rel_err

pytestmark = pytest.mark.gpu

ENUMS = dict(activation={"gelu": 0, "silu_gated": 1}, norm={"layernorm": 0, "rmsnorm": 1},
             norm_scope={"sequence": 0, "token": 1},
             weight_dtype={"f32": 0, "bf16": 1, "q8_0": 2, "q4_0": 3},
             kv_dtype={"f32": 0, "f16": 1, "bf16": 2})


def orc_cfg(orc, cfg):
    kw = {}
    for f in ("hidden_dim", "num_layers", "num_heads", "intermediate_dim", "vocab_size",
              "max_seq_len", "head_dim"):
        kw[f] = getattr(cfg, f)
    kw["use_bias"] = 1 if cfg.use_bias else 0
    kw["layer_norm_eps"] = cfg.layer_norm_eps
    for f, table in ENUMS.items():
        kw[f] = table[getattr(cfg, f)]
    return orc.default_config(**kw)


def small(**over):
    kw = dict(hidden_dim=64, num_layers=3, num_heads=4, intermediate_dim=96, vocab_size=211,
              max_seq_len=48)
    kw.update(over)
    return Transformer250MConfig(**kw)


def build(cfg, params):
    return TransformerModelPlugin().create_builder().build(cfg, parameters=params)


def test_plugin_identity():
    p = TransformerModelPlugin()  # MT:1127-1134
    assert p.id() == "transformer_model" and p.version() == (0, 1, 0)
    assert "transformer" in p.capabilities()


@pytest.mark.parametrize("use_bias", [True, False])
def test_forward_reference_mode_small(orc, use_bias):
    cfg = small(use_bias=use_bias)
    oc = orc_cfg(orc, cfg)
    params = orc.init_seeded(oc, 11)
    ids = orc.synth_ids(12, cfg.vocab_size, 19)
    model = build(cfg, params)
    assert model.name() == "TransformerModel" and model.num_parameters() == params.size
    got_all = model.forward_all(ids)
    got_last = model.forward(ids)
    rc, want_last, want_all = orc.forward(oc, params, ids, all_rows=True)
    assert rc == 0
    assert rel_err(got_all, want_all) < 1e-3 and rel_err(got_last, want_last) < 1e-3
    assert rel_err(got_last, got_all[-1]) < 1e-5
    assert np.array_equal(got_all.argmax(-1), want_all.argmax(-1))
    # the reference's own init (MT:604-611) through the default build path
    model2 = TransformerModelPlugin().create_builder().build(cfg)
    p_sin = orc.init_default(orc.num_parameters(oc), cfg.hidden_dim)
    rc, want_sin = orc.forward(oc, p_sin, [100, 200, 30])  # the shape of MT:1147-1149
    got_sin = model2.forward([100, 200, 30])
    assert got_sin.shape == (cfg.vocab_size,) and rel_err(got_sin, want_sin) < 1e-3


@pytest.mark.parametrize("over", [
    dict(norm_scope="token"),
    dict(norm_scope="token", norm="rmsnorm", activation="silu_gated", use_bias=False),
    dict(norm_scope="token", activation="silu_gated"),
    dict(norm_scope="token", head_dim=8),
    dict(norm="rmsnorm"),
])
def test_forward_extensions_f32(orc, over):
    cfg = small(**over)
    oc = orc_cfg(orc, cfg)
    params = orc.init_seeded(oc, 31)
    ids = orc.synth_ids(32, cfg.vocab_size, 17)
    got = build(cfg, params).forward_all(ids)
    rc, _, want = orc.forward(oc, params, ids, all_rows=True)
    assert rc == 0 and rel_err(got, want) < 1e-3
    assert np.array_equal(got.argmax(-1), want.argmax(-1))


@pytest.mark.parametrize("wd,kv", [("bf16", "bf16"), ("q8_0", "f16"), ("q4_0", "f16"), ("q4_0", "f32")])
@pytest.mark.parametrize("gated", [False, True])
def test_forward_low_precision(orc, wd, kv, gated):
    cfg = small(hidden_dim=128, intermediate_dim=256, num_heads=4, norm_scope="token",
                weight_dtype=wd, kv_dtype=kv, activation="silu_gated" if gated else "gelu",
                norm="rmsnorm" if gated else "layernorm", use_bias=not gated)
    oc = orc_cfg(orc, cfg)
    params = orc.init_seeded(oc, 41)
    ids = orc.synth_ids(42, cfg.vocab_size, 23)
    got = build(cfg, params).forward_all(ids)
    rc, _, want = orc.forward(oc, orc.apply_weight_dtype(oc, params), ids, all_rows=True)
    assert rc == 0 and rel_err(got, want) < 2e-2


@pytest.mark.parametrize("hd,wd,kv", [(64, "q8_0", "f16"), (128, "bf16", "bf16"), (128, "q4_0", "f16")])
def test_prefill_attention_on_matrix_cores(orc, hd, wd, kv):
    """Head dims 64 / 128 with a 16-bit cache take the matrix-core prefill attention: 150 rows
    (two query tiles, the second partial, key tiles with and without masking), then the same
    sequence in two chunks so that the second starts from a cached prefix (pos0 > 0)."""
    cfg = small(hidden_dim=2 * hd, num_heads=2, intermediate_dim=3 * hd, num_layers=2, max_seq_len=192,
                norm_scope="token", weight_dtype=wd, kv_dtype=kv)
    oc = orc_cfg(orc, cfg)
    params = orc.init_seeded(oc, 71)
    ids = orc.synth_ids(72, cfg.vocab_size, 150)
    rc, _, want = orc.forward(oc, orc.apply_weight_dtype(oc, params), ids, all_rows=True)
    model = build(cfg, params)
    got = model.forward_all(ids)
    assert rc == 0 and rel_err(got, want) < 2e-2
    s = model.session(batch=1, max_ctx=192)
    s.prefill(ids[:70], want_logits=False)
    last = s.prefill(ids[70:])
    assert rel_err(last[0], want[149]) < 2e-2


@pytest.mark.parametrize("hd,heads,wd,kv", [(64, 2, "q8_0", "f16"), (128, 2, "bf16", "bf16"), (64, 2, "bf16", "f32"),
                                            (64, 3, "q8_0", "f16"), (64, 3, "bf16", "bf16")])
def test_prompt_matmul_appends_to_the_cache(orc, hd, heads, wd, kv):
    """From 128 rows up the q|k|v matmul of a prompt pass writes keys and values into the cache
    itself: a second chunk of 140 rows behind a cached prefix of 130 (position offset > 0), and
    two sequences of 130 rows in one batch (rows of the second sequence), against the oracle.
    With 3 heads of 64 the query third ends inside a wave's 128-column block, which takes the
    matmul's general epilogue walk instead of the cache-append one."""
    cfg = small(hidden_dim=heads * hd, num_heads=heads, intermediate_dim=3 * hd, num_layers=2, max_seq_len=288,
                norm_scope="token", weight_dtype=wd, kv_dtype=kv, max_batch=2)
    oc = orc_cfg(orc, cfg)
    params = orc.init_seeded(oc, 73)
    pq = orc.apply_weight_dtype(oc, params)
    ids = orc.synth_ids(74, cfg.vocab_size, 270)
    other = orc.synth_ids(75, cfg.vocab_size, 130)
    rc, _, want = orc.forward(oc, pq, ids, all_rows=True)
    rc2, _, want_other = orc.forward(oc, pq, other, all_rows=True)
    assert rc == 0 and rc2 == 0
    model = build(cfg, params)
    s = model.session(batch=1, max_ctx=288)
    s.prefill(ids[:130], want_logits=False)
    last = s.prefill(ids[130:])
    assert rel_err(last[0], want[269]) < 2e-2
    step = s.decode(ids[:1])  # reads every cached position once more (two context splits)
    rc4, want_step = orc.forward(oc, pq, list(ids) + [int(ids[0])])
    assert rc4 == 0 and rel_err(step[0], want_step) < 2e-2
    s.close()
    s2 = model.session(batch=2, max_ctx=160)
    both = s2.prefill(np.stack([ids[:130], other]))
    assert rel_err(both[0], want[129]) < 2e-2 and rel_err(both[1], want_other[129]) < 2e-2
    # one more token per sequence: the decode step reads what the prompt pass cached
    rc3, _, want_next = orc.forward(oc, pq, list(other) + [5], all_rows=True)
    nxt = s2.decode(np.array([ids[130], 5], dtype=np.uint64))
    assert rc3 == 0 and rel_err(nxt[1], want_next[130]) < 2e-2 and rel_err(nxt[0], want[130]) < 2e-2
    s2.close()
    model.close()


def test_seeded_build_equals_uploaded_parameters(orc):
    cfg = small(norm_scope="token", weight_dtype="q4_0", hidden_dim=128, intermediate_dim=128)
    oc = orc_cfg(orc, cfg)
    ids = orc.synth_ids(7, cfg.vocab_size, 11)
    a = TransformerModelBuilder().build(cfg, seed=99).forward_all(ids)
    b = build(cfg, orc.init_seeded(oc, 99)).forward_all(ids)
    assert np.array_equal(a, b)


def test_errors_match_reference_messages(orc):
    cfg = small()
    model = build(cfg, orc.init_seeded(orc_cfg(orc, cfg), 1))
    with pytest.raises(ProcessingError, match=r"Token ID 211 out of range \[0, 210\]"):  # MT:817-821
        model.forward([1, 211])
    with pytest.raises(ProcessingError, match=r"Sequence length 49 out of range \[1, 48\]"):  # MT:798-801
        model.forward(list(range(49)))
    with pytest.raises(ProcessingError, match=r"Sequence length 0 out of range"):  # reference panics
        model.forward([])
    with pytest.raises(ConfigError):
        TransformerModelBuilder().build(small(hidden_dim=63))
    with pytest.raises(ProcessingError, match="Parameter access out of range"):  # MT:663-668
        build(cfg, np.zeros(1000, dtype=np.float32))
    with pytest.raises(ConfigError):
        model.session()  # whole-sequence norm cannot be cached


# ------------------------------------------------------------------ KV-cache sessions

@pytest.mark.parametrize("wd,kv,tol", [("f32", "f32", 1e-3), ("bf16", "bf16", 2e-2),
                                       ("q8_0", "f16", 2e-2), ("q4_0", "f16", 2e-2)])
def test_session_prefill_and_decode(orc, wd, kv, tol):
    cfg = small(hidden_dim=128, intermediate_dim=256, norm_scope="token", weight_dtype=wd,
                kv_dtype=kv, max_batch=4)
    oc = orc_cfg(orc, cfg)
    params = orc.init_seeded(oc, 51)
    pq = orc.apply_weight_dtype(oc, params)
    ids = orc.synth_ids(52, cfg.vocab_size, 20)
    _, _, want = orc.forward(oc, pq, ids, all_rows=True)
    model = build(cfg, params)
    s = model.session(batch=1, max_ctx=32)
    got = s.prefill(ids[:12])
    assert s.position == 12 and rel_err(got[0], want[11]) < tol
    for i in range(12, 20):
        step = s.decode(ids[i:i + 1])
        assert rel_err(step[0], want[i]) < tol, i
    assert s.position == 20
    with pytest.raises(ProcessingError):
        s.prefill(ids[:13])  # 20 + 13 > 32
    # chunked prefill continues from the cached prefix
    s.reset()
    s.prefill(ids[:5], want_logits=False)
    got2 = s.prefill(ids[5:12])
    assert rel_err(got2[0], want[11]) < tol


@pytest.mark.parametrize("wd", ["f32", "q4_0"])
def test_session_batch_equals_independent_sequences(orc, wd):
    cfg = small(hidden_dim=128, intermediate_dim=256, norm_scope="token", weight_dtype=wd,
                kv_dtype="f32" if wd == "f32" else "f16", max_batch=4)
    oc = orc_cfg(orc, cfg)
    params = orc.init_seeded(oc, 61)
    model = build(cfg, params)
    B, n = 3, 9
    ids = orc.synth_ids(62, cfg.vocab_size, B * (n + 4)).reshape(B, n + 4)
    sb = model.session(batch=B, max_ctx=32)
    lb = [sb.prefill(ids[:, :n])] + [sb.decode(ids[:, n + t]) for t in range(4)]
    for b in range(B):
        s1 = model.session(batch=1, max_ctx=32)
        l1 = [s1.prefill(ids[b, :n])] + [s1.decode(ids[b, n + t:n + t + 1]) for t in range(4)]
        # f32: the same arithmetic per row either way.  q4_0: a single sequence merges the norm
        # statistics inside the matmul, a batch of 3 at this width runs the norm kernel; the
        # activations are then rounded to f16, where a last-bit difference can flip a rounding
        tol = 1e-5 if wd == "f32" else 2e-4
        for t in range(5):
            assert rel_err(lb[t][b], l1[t][0]) < tol, (b, t)


@pytest.mark.parametrize("B", [5, 8, 16])
@pytest.mark.parametrize("wd,kv,norm,gated", [("q4_0", "f16", "layernorm", False), ("q4_0", "f16", "rmsnorm", True),
                                              ("q8_0", "bf16", "rmsnorm", False), ("q8_0", "f16", "layernorm", True),
                                              ("bf16", "bf16", "layernorm", False), ("f32", "f32", "rmsnorm", True)])
def test_session_large_batches_against_oracle(orc, B, wd, kv, norm, gated):
    """Batches of 5, 8 and 16 sequences pad to 8 / 16 accumulator rows in the decode matmul: the
    norm runs as a launch of its own from the producers' statistics records, the activations are
    staged without it, the residuals are fetched up front.  Widths of 160 and 288 are not multiples
    of the 128-wide groups of quantisation blocks (padded groups).  Every sequence's prompt logits, a few decode
    steps and the greedy tokens of the captured step are compared with the oracle's forward of
    that sequence alone, and the decode logits with a batch-1 session."""
    cfg = small(hidden_dim=160, num_heads=4, head_dim=32, intermediate_dim=288, num_layers=2, vocab_size=211,
                max_seq_len=40, norm_scope="token", weight_dtype=wd, kv_dtype=kv, norm=norm,
                activation="silu_gated" if gated else "gelu", use_bias=not gated, max_batch=16)
    tol = 1e-3 if wd == "f32" else 2e-2
    oc = orc_cfg(orc, cfg)
    params = orc.init_seeded(oc, 600 + B)
    pq = orc.apply_weight_dtype(oc, params)
    n, steps = 7, 4
    ids = orc.synth_ids(601 + B, cfg.vocab_size, B * (n + steps)).reshape(B, n + steps)
    want = [orc.forward(oc, pq, ids[b], all_rows=True)[2] for b in range(B)]
    model = build(cfg, params)
    sb = model.session(batch=B, max_ctx=40)
    lb = [sb.prefill(ids[:, :n])] + [sb.decode(ids[:, n + t]) for t in range(steps)]
    for b in range(B):
        for t in range(steps + 1):
            assert rel_err(lb[t][b], want[b][n - 1 + t]) < tol, (b, t)
    for b in (0, B // 2, B - 1):
        s1 = model.session(batch=1, max_ctx=40)
        l1 = [s1.prefill(ids[b, :n])] + [s1.decode(ids[b, n + t:n + t + 1]) for t in range(steps)]
        s1.close()
        for t in range(steps + 1):
            assert rel_err(lb[t][b], l1[t][0]) < (1e-5 if wd == "f32" else 2e-3), (b, t)
    # the captured greedy step at this batch: tokens equal the argmax of the stepwise logits
    sg, sl = model.session(batch=B, max_ctx=40), model.session(batch=B, max_ctx=40)
    first = sg.prefill(ids[:, :n]).argmax(-1).astype(np.uint64)
    sl.prefill(ids[:, :n])
    got = sg.decode_greedy(first, 6)
    tok = first
    for t in range(6):
        logits = sl.decode(tok)
        tok = logits.argmax(-1).astype(np.uint64)
        assert list(got[:, t]) == list(tok), t
    for x in (sb, sg, sl):
        x.close()
    model.close()


@pytest.mark.parametrize("heads,hd,wd,kv", [(2, 128, "q4_0", "f16"), (2, 128, "bf16", "bf16"),
                                            (4, 64, "q8_0", "bf16"), (4, 64, "f32", "f16")])
def test_decode_attention_many_splits_against_oracle(orc, heads, hd, wd, kv):
    """A session of 2048 positions with few heads splits the decode attention's context over 8
    workgroups per head (the in-kernel merge by the last split to finish).  A prompt of 2040
    tokens and 6 decode steps (the partial records are rewritten at the same addresses, the
    arrival counters reused) against the oracle's forward of the whole sequence, and against the
    prompt pass of the same prefix (matrix-core attention kernel)."""
    cfg = small(hidden_dim=256, num_heads=heads, head_dim=hd, intermediate_dim=384, num_layers=2, vocab_size=211,
                max_seq_len=2048, norm_scope="token", weight_dtype=wd, kv_dtype=kv)
    tol = 2e-2
    oc = orc_cfg(orc, cfg)
    params = orc.init_seeded(oc, 81)
    pq = orc.apply_weight_dtype(oc, params)
    n, steps = 2040, 6
    ids = orc.synth_ids(82, cfg.vocab_size, n + steps)
    rc, _, want = orc.forward(oc, pq, ids, all_rows=True)
    assert rc == 0
    model = build(cfg, params)
    s = model.session(batch=1, max_ctx=2048)
    first = s.prefill(ids[:n])[0]
    assert rel_err(first, want[n - 1]) < tol
    dec = [s.decode(ids[n + t:n + t + 1])[0] for t in range(steps)]
    for t in range(steps):
        assert rel_err(dec[t], want[n + t]) < tol, t
        assert int(dec[t].argmax()) == int(want[n + t].argmax()) or \
            np.sort(want[n + t])[-1] - np.sort(want[n + t])[-2] < 1e-3 * np.abs(want[n + t]).max()
    s2 = model.session(batch=1, max_ctx=2048)
    again = s2.prefill(ids[:n + steps])[0]  # the last decode step's logits, from the prompt pass
    assert rel_err(dec[-1], again) < tol
    # the captured greedy step on the same split attention
    s2.reset()
    s2.prefill(ids[:n], want_logits=False)
    tok = np.array([ids[n]], dtype=np.uint64)
    got = s2.decode_greedy(tok, 4)[0]
    s.reset()
    s.prefill(ids[:n], want_logits=False)
    for t in range(4):
        logits = s.decode(tok)
        tok = logits.argmax(-1).astype(np.uint64)
        assert int(got[t]) == int(tok[0]), t
    s.close()
    s2.close()
    model.close()


def test_greedy_decode_matches_oracle_token_for_token(orc):
    cfg = small(norm_scope="token", max_batch=2)
    oc = orc_cfg(orc, cfg)
    params = orc.init_seeded(oc, 71)
    model = build(cfg, params)
    prompt = orc.synth_ids(72, cfg.vocab_size, 10)
    # oracle: prefill, then 12 greedy steps
    so = orc.Session(oc, params, 48)
    _, last = so.feed(prompt)
    want = []
    tok = int(last.argmax())
    first = tok
    for _ in range(12):
        _, l = so.feed([tok])
        tok = int(l.argmax())
        want.append(tok)
    s = model.session(batch=2, max_ctx=48)
    logits = s.prefill(np.stack([prompt, prompt]))
    assert int(logits[0].argmax()) == first
    got = s.decode_greedy([first, first], 12)
    assert got.shape == (2, 12) and list(got[0]) == want and list(got[1]) == want
    assert s.position == 22
    # a second replay of the captured step continues correctly
    more = s.decode_greedy(got[:, -1], 5)
    for _ in range(5):
        _, l = so.feed([tok])
        tok = int(l.argmax())
        want.append(tok)
    assert list(more[0]) == want[12:]


@pytest.mark.parametrize("vocab", [211, 1003, 1024, 4099])
def test_device_argmax_rows_of_any_alignment(orc, vocab):
    """The on-device greedy step (argmax kernel: 16-byte loads over the aligned middle of each
    logits row) against the host's argmax of the same step's logits, for three different sequences
    in one batch: with an odd vocabulary rows 1 and 2 start off a 16-byte boundary."""
    cfg = small(norm_scope="token", max_batch=3, vocab_size=vocab)
    oc = orc_cfg(orc, cfg)
    params = orc.init_seeded(oc, 300 + vocab)
    model = build(cfg, params)
    prompts = np.stack([orc.synth_ids(301 + b, vocab, 9) for b in range(3)])
    a, b = model.session(batch=3, max_ctx=40), model.session(batch=3, max_ctx=40)
    first = a.prefill(prompts).argmax(-1).astype(np.uint64)
    b.prefill(prompts)
    got = a.decode_greedy(first, 10)
    tok = first
    for t in range(10):
        logits = b.decode(tok)
        tok = logits.argmax(-1).astype(np.uint64)  # numpy: lowest index among equal maxima, like the kernel
        assert list(got[:, t]) == list(tok), t
    a.close()
    b.close()
    model.close()


# ------------------------------------------------------------------ the default 250M configuration, full size

def test_config1_full_size_f32(orc):
    """Transformer250MConfig::default(), seeded N(0, 0.02)-like weights, 128 uniform ids."""
    cfg = Transformer250MConfig()
    oc = orc_cfg(orc, cfg)
    params = orc.init_seeded(oc, 0xC0E05)
    ids = orc.synth_ids(0xC0E06, cfg.vocab_size, 128)
    model = build(cfg, params)
    n = model.num_parameters()
    assert 160_000_000 < n < 170_000_000  # MT:1143-1144
    got = model.forward(ids)
    assert got.shape == (50257,)  # MT:1149
    rc, want = orc.forward(oc, params, ids)
    assert rc == 0
    top = np.sort(want)[::-1]
    print("config1: rel err", rel_err(got, want), "top-2 gap", top[0] - top[1], flush=True)
    assert rel_err(got, want) < 1e-3
    assert int(got.argmax()) == int(want.argmax())
    # "full-sequence logits": every one of the 128 rows against the oracle's, not only the last
    got_all = model.forward_all(ids)
    rc, want_last, want_all = orc.forward(oc, params, ids, all_rows=True)
    assert rc == 0 and got_all.shape == want_all.shape == (128, 50257)
    assert np.array_equal(want_all[-1], want_last)
    row_err = np.abs(got_all.astype(np.float64) - want_all).max(-1) / np.abs(want_all).max(-1)
    print("config1 all rows: worst row rel err", row_err.max(), flush=True)
    assert row_err.max() < 1e-3
    assert np.array_equal(got_all.argmax(-1), want_all.argmax(-1))
    assert rel_err(got_all[-1], got) < 1e-5
    # the reference's unit test (MT:1137-1150) on the default sin init
    model.close()
    model2 = TransformerModelBuilder().build(cfg)
    out = model2.forward([100, 200, 300])
    p_sin = orc.init_default(orc.num_parameters(oc), 768)
    rc, want2 = orc.forward(oc, p_sin, [100, 200, 300])
    assert out.shape == (50257,) and rel_err(out, want2) < 1e-3


# ------------------------------------------------------------------ the larger benchmark configurations, full size
# The CPU oracle needs minutes to hours per token at these sizes, so the full-size checks use
# properties that do not depend on size: the prompt pass (matrix-core matmuls and attention on
# all rows) and the decode path (streaming matmuls, split-context attention, folded norms, graph
# replay) are two independent implementations of the same function and must agree on the logits
# of every position; sequences in a batch must not influence each other.  Each configuration runs
# at the context and batch it is specified with.

# name -> (config, prompt tokens, decode steps, batch)
FULL = {
    # 250M bf16: prefill 512, then 256 greedy steps at batch 1 (cache grows to 768)
    "cfg2-250m-bf16": (dict(norm_scope="token", weight_dtype="bf16", kv_dtype="bf16", max_batch=4), 512, 256, 2),
    # 250M Q8_0: decode at batch 1 and 8, context 2048
    "cfg3-250m-q8_0": (dict(max_seq_len=2048, norm_scope="token", weight_dtype="q8_0", kv_dtype="f16",
                            max_batch=8), 2036, 12, 8),
    # 1B Q4_0, 16 heads of 64: prefill 2048 tokens at batch 4, then 128 decode steps
    "cfg4-1b-q4_0": (dict(hidden_dim=2048, num_layers=24, num_heads=16, head_dim=64, intermediate_dim=8192,
                          vocab_size=32000, max_seq_len=2176, norm_scope="token", weight_dtype="q4_0",
                          kv_dtype="f16", max_batch=4), 2048, 128, 4),
    # 7B Q4_0: decode at batch 1 and 16, context 4096, f16 cache
    "cfg5-7b-q4_0": (dict(hidden_dim=4096, num_layers=32, num_heads=32, head_dim=128, intermediate_dim=11008,
                          vocab_size=32000, max_seq_len=4096, use_bias=False, activation="silu_gated",
                          norm="rmsnorm", norm_scope="token", weight_dtype="q4_0", kv_dtype="f16",
                          max_batch=16), 4084, 12, 16),
}


def _same_token_or_near_tie(got, want):
    top = np.sort(want)
    return int(got.argmax()) == int(want.argmax()) or top[-1] - top[-2] < 1e-3 * np.abs(want).max()


@pytest.mark.parametrize("name", sorted(FULL))
def test_full_size_prefill_and_decode_agree(name):
    kw, n_prompt, n_dec, B = FULL[name]
    cfg = Transformer250MConfig(**kw)
    ctx = n_prompt + n_dec
    model = TransformerModelBuilder().build(cfg, seed=0xC0E05)
    rng = np.random.default_rng(0xC0E06)
    seqs = rng.integers(0, cfg.vocab_size, (B, ctx), dtype=np.uint64)
    ids = seqs[0]
    checks = sorted({0, n_dec // 2, n_dec - 1})
    # batch 1: the decode path's logits at the first, a middle and the last step ...
    s = model.session(batch=1, max_ctx=ctx)
    first = s.prefill(ids[:n_prompt])[0]
    dec = {}
    for t in range(n_dec):
        l = s.decode(ids[n_prompt + t:n_prompt + t + 1])
        if t in checks:
            dec[t] = l[0].copy()
    assert s.position == ctx
    s.close()
    assert np.isfinite(first).all()
    # ... against one prompt pass over the prefix ending at the token that step fed
    worst = 0.0
    s2 = model.session(batch=1, max_ctx=ctx)
    for t in checks:
        s2.reset()
        want = s2.prefill(ids[:n_prompt + t + 1])[0]
        err = rel_err(dec[t], want)
        worst = max(worst, err)
        assert err < 2e-2, (name, t, err)
        assert _same_token_or_near_tie(dec[t], want), (name, t)
    # the captured greedy step (one graph replay per token) against the stepwise decode
    s2.reset()
    l0 = s2.prefill(ids[:n_prompt])
    tok = l0.argmax(-1).astype(np.uint64)
    s3 = model.session(batch=1, max_ctx=ctx)
    s3.prefill(ids[:n_prompt], want_logits=False)
    k = min(n_dec, 8)
    greedy = s3.decode_greedy(tok, k)[0]
    for t in range(k):
        tok = s2.decode(tok).argmax(-1).astype(np.uint64)
        assert int(greedy[t]) == int(tok[0]), (name, t)
    s2.close()
    s3.close()
    print(name, "batch 1, context", ctx, ": decode vs prompt pass, worst rel err", worst, flush=True)

    # batch B at the same context: B different sequences in one session (prompt pass over B x
    # n_prompt rows, then every decode step at batch B) against some of them alone
    sb = model.session(batch=B, max_ctx=ctx)
    lb = sb.prefill(seqs[:, :n_prompt])
    db = {}
    for t in range(n_dec):
        l = sb.decode(seqs[:, n_prompt + t])
        if t in checks:
            db[t] = l.copy()
    assert sb.position == ctx
    worst_b = 0.0
    for b in sorted({0, B // 2, B - 1}):
        s1 = model.session(batch=1, max_ctx=ctx)
        l1 = s1.prefill(seqs[b, :n_prompt])
        assert rel_err(lb[b], l1[0]) < 2e-2, (name, b)
        for t in range(n_dec):
            d1 = s1.decode(seqs[b, n_prompt + t:n_prompt + t + 1])
            if t in checks:
                err = rel_err(db[t][b], d1[0])
                worst_b = max(worst_b, err)
                assert err < 2e-2, (name, b, t, err)
                assert _same_token_or_near_tie(db[t][b], d1[0]), (name, b, t)
        s1.close()
    # the captured greedy step at batch B against the stepwise decode of the same session state
    sb.reset()
    tok = sb.prefill(seqs[:, :n_prompt]).argmax(-1).astype(np.uint64)
    sg = model.session(batch=B, max_ctx=ctx)
    sg.prefill(seqs[:, :n_prompt], want_logits=False)
    k = min(n_dec, 6)
    greedy = sg.decode_greedy(tok, k)
    for t in range(k):
        tok = sb.decode(tok).argmax(-1).astype(np.uint64)
        assert list(greedy[:, t]) == list(tok), (name, t)
    sg.close()
    sb.close()
    print(name, "batch", B, "context", ctx, ": rows vs the same rows alone, worst rel err", worst_b, flush=True)
    model.close()


@pytest.mark.parametrize("wd,n", [("q4_0", 40), ("q8_0", 17), ("q4_0", 64)])
def test_short_prompt_equals_decode_steps(wd, n):
    """Prompts of up to 64 rows on quantised weights run on the matmul that streams the quantised
    blocks (7B-wide layers, 17 / 40 / 64 rows: one, three and four fragments of 16 rows, the cache
    written by the append kernel).  Feeding the same tokens one at a time through the decode path
    (streaming matmuls on f16 activations, split-context attention) must give the same logits."""
    cfg = Transformer250MConfig(hidden_dim=4096, num_layers=2, num_heads=32, head_dim=128, intermediate_dim=11008,
                                vocab_size=2000, max_seq_len=128, use_bias=False, activation="silu_gated",
                                norm="rmsnorm", norm_scope="token", weight_dtype=wd, kv_dtype="f16")
    model = TransformerModelBuilder().build(cfg, seed=21)
    ids = np.random.default_rng(22).integers(0, cfg.vocab_size, n, dtype=np.uint64)
    a = model.session(batch=1, max_ctx=128)
    want = a.prefill(ids)[0]
    nxt = a.decode(np.array([3], dtype=np.uint64))[0]
    a.close()
    b = model.session(batch=1, max_ctx=128)
    for t in range(n):
        got = b.decode(ids[t:t + 1])[0]
    nxt_b = b.decode(np.array([3], dtype=np.uint64))[0]
    b.close()
    model.close()
    assert rel_err(want, got) < 2e-2 and int(want.argmax()) == int(got.argmax())
    assert rel_err(nxt, nxt_b) < 2e-2  # the step after reads the cache each path wrote


def test_long_prompt_in_one_pass_equals_chunks():
    """2900 rows through a 2048-wide layer: the q|k|v matmul is 12 x 24 = 256 + 32 tiles, so the
    tiles of its last round are split along k and the cache is written by the kernel that sums
    them; FFN-up (12 x 16 tiles) has every tile split.  The same prompt fed in chunks of 700 rows
    runs those matmuls with other launch shapes (and reads the earlier chunks back from the cache):
    the logits after the last token must agree, and so must a decode step on top of either."""
    cfg = Transformer250MConfig(hidden_dim=2048, num_layers=1, num_heads=16, head_dim=128, intermediate_dim=4096,
                                vocab_size=1000, max_seq_len=3000, norm_scope="token", weight_dtype="bf16",
                                kv_dtype="f16", activation="silu_gated", norm="rmsnorm", use_bias=False)
    model = TransformerModelBuilder().build(cfg, seed=11)
    ids = np.random.default_rng(12).integers(0, cfg.vocab_size, 2900, dtype=np.uint64)
    one = model.session(batch=1, max_ctx=3000)
    l_one = one.prefill(ids)[0]
    d_one = one.decode(np.array([7], dtype=np.uint64))[0]
    one.close()
    ch = model.session(batch=1, max_ctx=3000)
    for lo in range(0, 2900, 700):
        l_ch = ch.prefill(ids[lo:lo + 700])[0]
    d_ch = ch.decode(np.array([7], dtype=np.uint64))[0]
    ch.close()
    model.close()
    assert np.isfinite(l_one).all() and rel_err(l_one, l_ch) < 2e-3 and rel_err(d_one, d_ch) < 2e-3
    assert int(l_one.argmax()) == int(l_ch.argmax())


def test_rustllm_file_round_trip_through_the_model(orc, tmp_path):
    """write_to -> load reproduces the logits; the same file loaded as Q4_0 stays within the
    quantised bar of the oracle on the quantised weights."""
    cfg = small(norm_scope="token")
    oc = orc_cfg(orc, cfg)
    params = orc.init_seeded(oc, 91)
    ids = orc.synth_ids(92, cfg.vocab_size, 17)
    model = build(cfg, params)
    want = model.forward(ids)
    path = tmp_path / "small.rustllm"
    model.write_to(path)
    again = TransformerModelBuilder().load(path)
    assert again.config().intermediate_dim == cfg.intermediate_dim and again.config().norm_scope == "token"
    assert np.array_equal(again.forward(ids), want)
    q = TransformerModelBuilder().load(path, weight_dtype="q4_0", kv_dtype="f16")
    qc = orc_cfg(orc, q.config())
    rc, ref = orc.forward(qc, orc.apply_weight_dtype(qc, params), ids)
    assert rc == 0 and rel_err(q.forward(ids), ref) < 2e-2
    with pytest.raises(ProcessingError):
        TransformerModelBuilder().build(cfg, seed=3).write_to(path)


# ------------------------------------------------------------------ Model: Send + Sync (CM:77)

def test_two_threads_share_a_model_and_a_session(orc):
    """The reference's model is Send + Sync and forward(&self) is re-entrant; the library
    serialises calls on one handle instead.  Two threads call forward on one model at the same
    time (ctypes releases the interpreter lock during the call) and get the logits of a serial
    run, bit for bit; two threads step ONE session k times each and both succeed, the position
    having advanced by 2k (the bound is checked under the same lock that advances it)."""
    import threading

    cfg = small(hidden_dim=128, intermediate_dim=256, norm_scope="token", weight_dtype="q4_0", kv_dtype="f16",
                max_seq_len=96)
    oc = orc_cfg(orc, cfg)
    params = orc.init_seeded(oc, 91)
    model = build(cfg, params)
    seqs = [orc.synth_ids(92 + i, cfg.vocab_size, 40 + i) for i in range(2)]
    serial = [model.forward_all(s) for s in seqs]
    out, errs = {}, []

    def fwd(i):
        try:
            for _ in range(20):
                out[i] = model.forward_all(seqs[i])
                assert np.array_equal(out[i], serial[i])
        except Exception as e:  # noqa: BLE001
            errs.append(e)

    ts = [threading.Thread(target=fwd, args=(i,)) for i in range(2)]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    assert not errs, errs
    assert all(np.array_equal(out[i], serial[i]) for i in range(2))

    s = model.session(batch=1, max_ctx=96)
    s.prefill(seqs[0][:10], want_logits=False)
    k = 30

    def step():
        try:
            for _ in range(k):
                assert np.isfinite(s.decode(np.array([7], dtype=np.uint64))).all()
        except Exception as e:  # noqa: BLE001
            errs.append(e)

    ts = [threading.Thread(target=step) for _ in range(2)]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    assert not errs, errs
    assert s.position == 10 + 2 * k
    # the 60 interleaved steps all fed token 7: the cache equals that of a serial run
    s1 = model.session(batch=1, max_ctx=96)
    s1.prefill(seqs[0][:10], want_logits=False)
    for _ in range(2 * k):
        last = s1.decode(np.array([7], dtype=np.uint64))
    a = s.decode(np.array([9], dtype=np.uint64))
    b = s1.decode(np.array([9], dtype=np.uint64))
    assert np.array_equal(a, b) and last.shape == a.shape
    s.close()
    s1.close()
    model.close()


# ------------------------------------------------------------------ a sweep over the configuration space

def _sweep_configs():
    """24 small configurations drawn from the whole space the ABI accepts (fixed seed): widths that
    are and are not multiples of the kernels' tile sizes, one to four layers, decoupled head sizes,
    every weight / cache type, both norms, both feed-forward shapes, with and without biases."""
    rng = np.random.default_rng(20240607)
    out = []
    for i in range(24):
        wd = ["f32", "bf16", "q8_0", "q4_0"][i % 4]
        quant = wd in ("q8_0", "q4_0")
        unit = 32 if quant else 8
        heads = int(rng.choice([1, 2, 3, 4, 6]))
        hd = int(rng.choice([8, 16, 32, 64, 128])) if not quant else int(rng.choice([32, 64, 128]))
        decoupled = bool(rng.integers(0, 2)) or quant
        hidden = int(rng.integers(1, 7)) * unit * (1 if decoupled else heads)
        if not decoupled:
            hd = hidden // heads
        inter = int(rng.integers(1, 9)) * unit
        kv = ["f32", "f16", "bf16"][int(rng.integers(0, 3))]
        out.append(dict(hidden_dim=hidden, num_layers=int(rng.integers(1, 5)), num_heads=heads,
                        head_dim=hd if decoupled else 0, intermediate_dim=inter,
                        vocab_size=int(rng.integers(17, 400)), max_seq_len=64,
                        norm_scope="token", weight_dtype=wd, kv_dtype=kv,
                        norm=["layernorm", "rmsnorm"][int(rng.integers(0, 2))],
                        activation=["gelu", "silu_gated"][int(rng.integers(0, 2))],
                        use_bias=bool(rng.integers(0, 2)), max_batch=4))
    return out


@pytest.mark.parametrize("idx", range(24))
def test_configuration_sweep_against_oracle(orc, idx):
    """forward_all, a chunked prompt pass, decode steps (batch 1 and 3) and greedy tokens of one
    drawn configuration against the oracle's forward of the same parameters."""
    kw = _sweep_configs()[idx]
    cfg = Transformer250MConfig(**kw)
    tol = 1e-3 if kw["weight_dtype"] == "f32" and kw["kv_dtype"] == "f32" else 2e-2
    oc = orc_cfg(orc, cfg)
    params = orc.init_seeded(oc, 5000 + idx)
    pq = orc.apply_weight_dtype(oc, params)
    n, steps, B = 21, 5, 3
    ids = orc.synth_ids(6000 + idx, cfg.vocab_size, B * (n + steps)).reshape(B, n + steps)
    want = [orc.forward(oc, pq, ids[b], all_rows=True)[2] for b in range(B)]
    model = build(cfg, params)
    got = model.forward_all(ids[0])
    assert rel_err(got, want[0]) < tol, kw
    s = model.session(batch=1, max_ctx=40)
    s.prefill(ids[0, :8], want_logits=False)
    l = s.prefill(ids[0, 8:n])
    assert rel_err(l[0], want[0][n - 1]) < tol, kw
    for t in range(steps):
        l = s.decode(ids[0, n + t:n + t + 1])
        assert rel_err(l[0], want[0][n + t]) < tol, (kw, t)
    sb = model.session(batch=B, max_ctx=40)
    lb = sb.prefill(ids[:, :n])
    for b in range(B):
        assert rel_err(lb[b], want[b][n - 1]) < tol, (kw, b)
    for t in range(steps):
        lb = sb.decode(ids[:, n + t])
        for b in range(B):
            assert rel_err(lb[b], want[b][n + t]) < tol, (kw, b, t)
    # the captured greedy step against the stepwise logits of the same state
    sg = model.session(batch=B, max_ctx=40)
    first = sg.prefill(ids[:, :n]).argmax(-1).astype(np.uint64)
    sb.reset()
    sb.prefill(ids[:, :n], want_logits=False)
    toks = sg.decode_greedy(first, 4)
    tok = first
    for t in range(4):
        tok = sb.decode(tok).argmax(-1).astype(np.uint64)
        assert list(toks[:, t]) == list(tok), (kw, t)
    for x in (s, sb, sg):
        x.close()
    model.close()


# ------------------------------------------------------------------ graph replay switched off from outside

def test_graph_replay_is_refused_when_switched_off_from_outside():
    """With COEUS_NO_GRAPH=1 (the switch that a loaded profiler tool library also throws) a session
    launches its greedy steps kernel by kernel, refuses set_graph(True), and generates the same ids
    as a session of a plain process that replays its captured graph."""
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = """
import json, numpy as np
from coeus_amd import ProcessingError, Transformer250MConfig, TransformerModelPlugin
cfg = Transformer250MConfig(hidden_dim=256, num_layers=2, num_heads=4, intermediate_dim=512, vocab_size=1000,
                            max_seq_len=64, norm_scope="token", weight_dtype="q4_0", kv_dtype="f16")
m = TransformerModelPlugin().create_builder().build(cfg, seed=5)
s = m.session(batch=1, max_ctx=64)
refused = False
try:
    s.set_graph(True)
except ProcessingError as e:
    refused = "graph replay refused" in str(e)
last = s.prefill(np.arange(20, dtype=np.uint64) * 7 % 1000)
ids = s.decode_greedy(last.argmax(-1).astype(np.uint64), 12)
ms, launches, nbytes = s.time_decode_matmuls(2)
print(json.dumps({"graph": s.graph_enabled, "refused": refused, "ids": ids[0].tolist(), "launches": launches}))
"""
    res = {}
    for name, extra in (("plain", {}), ("off", {"COEUS_NO_GRAPH": "1"})):
        env = {k: v for k, v in os.environ.items() if k != "COEUS_NO_GRAPH"}
        env.update(extra)
        out = subprocess.run([sys.executable, "-c", code], env=env, cwd=root, capture_output=True, text=True, timeout=110)
        assert out.returncode == 0, out.stderr[-800:]
        res[name] = json.loads(out.stdout.strip().splitlines()[-1])
    assert res["plain"]["graph"] is True and res["plain"]["refused"] is False
    assert res["off"]["graph"] is False and res["off"]["refused"] is True
    assert res["plain"]["ids"] == res["off"]["ids"] and res["off"]["launches"] == 2 * (4 * 2 + 1)
