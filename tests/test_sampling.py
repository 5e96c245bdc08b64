"""Token sampling.  The reference names the knobs (BasicGenerationConfig, core/model.rs:718-753) but
has no sampler, so the oracle's orc_sample is the specification; it is pinned here by what the
mathematics fixes rather than by a second copy of its code:
  * its exponential against libm on the whole useful range;
  * temperature -> 0, top_k = 1 and a dominant logit all reduce to argmax (lowest index on ties);
  * the empirical distribution over many seeds matches softmax(z / T) restricted to the top-k /
    nucleus set (chi-square style bound), and tokens outside the set are never drawn;
  * the draw depends on (seed, position, row) only.
The GPU tests then require the device sampler to return exactly the oracle's token."""
import math

import numpy as np
import pytest


def softmax(z, t):
    z = np.asarray(z, np.float64) / t
    e = np.exp(z - z.max())
    return e / e.sum()


def test_exponential_matches_libm(orc):
    xs = np.concatenate([-np.logspace(-6, math.log10(86.9), 4000), [0.0, -1e-9, -86.99, -87.0, -200.0]])
    for x in xs:
        got, want = orc.exp_nonpositive(x), math.exp(np.float32(x)) if x > -87.0 else 0.0
        assert abs(got - want) <= 3e-7 * want + 1e-45, x
    assert orc.exp_nonpositive(0.0) == 1.0


def test_reductions_to_argmax(orc):
    rng = np.random.default_rng(1)
    z = rng.standard_normal(500).astype(np.float32)
    z[[17, 300]] = z.max() + 1.0  # a tie: the lower index wins
    for kw in (dict(temperature=0.0), dict(temperature=-1.0), dict(top_k=1, temperature=0.7),
               dict(top_k=1, top_p=0.3, temperature=5.0)):
        for seed in range(20):
            assert orc.sample(z, seed=seed, **kw) == 17
    big = z.copy()
    big[123] = 200.0  # every other weight rounds to zero
    for seed in range(20):
        assert orc.sample(big, temperature=1.0, seed=seed) == 123
        assert orc.sample(big, temperature=1.0, top_k=40, seed=seed) == 123


@pytest.mark.parametrize("top_k,top_p,t", [(0, 0.0, 1.0), (0, 0.0, 0.5), (8, 0.0, 1.3), (16, 0.6, 1.0), (64, 0.9, 0.8)])
def test_distribution(orc, top_k, top_p, t):
    rng = np.random.default_rng(2)
    z = (rng.standard_normal(40) * 1.5).astype(np.float32)
    p = softmax(z, t)
    order = np.lexsort((np.arange(z.size), -z))  # value descending, index ascending
    allowed = order[:top_k] if top_k else np.arange(z.size)
    if top_k and 0 < top_p < 1:
        cum = np.cumsum(p[allowed]) / p[allowed].sum()
        allowed = allowed[:int(np.searchsorted(cum, top_p - 1e-6) + 1)]
    q = np.zeros_like(p)
    q[allowed] = p[allowed] / p[allowed].sum()
    n = 40_000
    counts = np.bincount([orc.sample(z, top_k, top_p, t, seed=s, position=s % 7, row=s % 3) for s in range(n)],
                         minlength=z.size)
    assert counts[q == 0].sum() == 0
    sd = np.sqrt(n * q * (1 - q)) + 1.0
    assert np.all(np.abs(counts - n * q) < 5 * sd), (counts, n * q)


def test_nan_logits_are_never_chosen(orc):
    z = np.random.default_rng(4).standard_normal(300).astype(np.float32)
    z[::2] = np.nan
    z[41] = 9.0
    for kw in (dict(temperature=0.0), dict(top_k=1, temperature=1.0)):
        assert orc.sample(z, seed=1, **kw) == 41
    for seed in range(200):
        for kw in (dict(temperature=1.5), dict(temperature=1.5, top_k=64), dict(temperature=2.0, top_k=30, top_p=0.8)):
            assert orc.sample(z, seed=seed, **kw) % 2 == 1
    nothing = np.full(50, np.nan, dtype=np.float32)
    for kw in (dict(temperature=0.0), dict(temperature=1.0), dict(temperature=1.0, top_k=8), dict(temperature=1.0, top_k=8, top_p=0.5)):
        assert orc.sample(nothing, seed=3, **kw) == 0


def test_draw_is_a_function_of_seed_position_row(orc):
    z = np.random.default_rng(3).standard_normal(1000).astype(np.float32)
    a = [orc.sample(z, 0, 0, 1.0, seed=9, position=p, row=r) for p in range(6) for r in range(4)]
    b = [orc.sample(z, 0, 0, 1.0, seed=9, position=p, row=r) for p in range(6) for r in range(4)]
    c = [orc.sample(z, 0, 0, 1.0, seed=10, position=p, row=r) for p in range(6) for r in range(4)]
    assert a == b and a != c and len(set(a)) > 6
    u = [orc.sample_u24(5, p, 0) for p in range(4000)]
    assert 0 <= min(u) and max(u) < 1 << 24 and abs(np.mean(u) / (1 << 24) - 0.5) < 0.02


@pytest.mark.gpu
@pytest.mark.parametrize("vocab", [211, 32000, 50257])
def test_device_sampler_equals_the_specification(orc, vocab):
    import ctypes as C

    from coeus_amd import _lib
    from coeus_amd.device import DeviceArray, synchronize
    from coeus_amd.plugin import _check

    lib = _lib.load()
    rng = np.random.default_rng(vocab)
    rows = 7
    z = (rng.standard_normal((rows, vocab)) * 2.0).astype(np.float32)
    z[1, [3, 77, 200]] = z[1].max() + 0.5   # ties at the top
    z[2] = np.round(z[2])                   # many ties everywhere
    z[3, 5] = 60.0                          # one dominant token
    z[5] = np.nan                           # nothing to choose from: index 0
    z[6, ::3] = np.nan                      # NaN entries (the first one included) are never chosen
    dz, out = DeviceArray.from_host(z), DeviceArray((rows,), np.uint64)
    for top_k, top_p, t in [(0, 0.0, 1.0), (0, 0.0, 0.3), (1, 0.0, 1.0), (7, 0.0, 1.7), (40, 0.0, 1.0),
                            (64, 0.0, 0.9), (40, 0.5, 1.0), (64, 0.95, 1.2), (5, 0.01, 1.0), (0, 0.0, 0.0)]:
        for seed, pos in [(0, 0), (1, 17), (123456789, 4095)]:
            cfg = _lib.CSampling(t, top_k, top_p, seed)
            _check(lib.coeus_op_sample(dz.ptr, rows, vocab, C.byref(cfg), pos, out.ptr, None))
            synchronize()
            got = out.to_host()
            want = [orc.sample(z[r], top_k, top_p, t, seed, pos, r) for r in range(rows)]
            assert list(got) == want, (top_k, top_p, t, seed, pos)


@pytest.mark.gpu
def test_generate_matches_stepwise_oracle_sampling(orc):
    """Session.generate: every drawn token equals the specification applied to the device's own
    logits of that step (decode() exposes them), so the loop, the position keying and the history
    are checked without depending on last-bit agreement of the logits with the CPU."""
    from coeus_amd import BasicGenerationConfig, Transformer250MConfig, TransformerModelBuilder

    cfg = Transformer250MConfig(hidden_dim=64, num_layers=2, num_heads=4, intermediate_dim=96, vocab_size=211,
                                max_seq_len=64, norm_scope="token", max_batch=2)
    model = TransformerModelBuilder().build(cfg, seed=5)
    prompt = np.array([[1, 2, 3, 4, 5], [9, 8, 7, 6, 5]], dtype=np.uint64)
    s = model.session(batch=2, max_ctx=64)
    first = s.prefill(prompt).argmax(-1).astype(np.uint64)
    got = s.generate(first, 12, temperature=0.9, top_k=20, top_p=0.9, seed=77)
    s2 = model.session(batch=2, max_ctx=64)
    s2.prefill(prompt)
    tok = first
    for step in range(12):
        logits = s2.decode(tok)
        pos = prompt.shape[1] + step + 1  # the position the drawn token takes
        tok = np.array([orc.sample(logits[b], 20, 0.9, 0.9, 77, pos, b) for b in range(2)], dtype=np.uint64)
        assert list(got[:, step]) == list(tok), step
    out = model.generate([1, 2, 3], BasicGenerationConfig(max_length=8, temperature=0.0))
    s3 = model.session(batch=1, max_ctx=64)
    g = s3.prefill(np.array([[1, 2, 3]], dtype=np.uint64)).argmax(-1).astype(np.uint64)
    assert out == [int(g[0])] + [int(t) for t in s3.decode_greedy(g, 7)[0]]
    assert len(model.generate([1, 2, 3], BasicGenerationConfig(max_length=5, temperature=1.0, top_k=10), seed=3)) == 5
