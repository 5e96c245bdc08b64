"""An independent float64 numpy implementation of the transformer forward.

Written from the mathematical definition (vectorised, whole-matrix operations), not from the
oracle's loops, so that it can arbitrate: the oracle and the HIP path are both compared with it.
Supports the reference semantics (whole-slice LayerNorm, MT:105-128) and the extension switches.
"""
import numpy as np


def head_dim(cfg):
    return cfg.head_dim or cfg.hidden_dim // cfg.num_heads


def offsets(cfg):
    """Flat-buffer offsets derived independently from MT:677-740 / MT:839-880."""
    H, I, V = cfg.hidden_dim, cfg.intermediate_dim, cfg.vocab_size
    inner = cfg.num_heads * head_dim(cfg)
    gated = cfg.activation == 1
    names = [("ln1_s", H), ("ln1_b", H), ("wq", H * inner), ("wk", H * inner),
             ("wv", H * inner), ("wo", inner * H)]
    if cfg.use_bias:
        names += [("bq", inner), ("bk", inner), ("bv", inner), ("bo", H)]
    names += [("ln2_s", H), ("ln2_b", H)]
    if gated:
        names += [("w_gate", H * I)]
    names += [("w_up", H * I), ("w_down", I * H)]
    if cfg.use_bias:
        if gated:
            names += [("b_gate", I)]
        names += [("b_up", I), ("b_down", H)]
    rel, o = {}, 0
    for n, sz in names:
        rel[n] = (o, sz)
        o += sz
    return V * H, o, rel


def pe_table(S, H):
    pos = np.arange(S, dtype=np.float64)[:, None]
    i = np.arange(H // 2, dtype=np.float64)[None, :]
    ang = pos / np.power(10000.0, 2.0 * i / H)
    t = np.zeros((S, H))
    t[:, 0:2 * (H // 2):2] = np.sin(ang)
    t[:, 1:2 * (H // 2):2] = np.cos(ang)
    return t


def norm(cfg, x, scale, bias):
    axis = None if cfg.norm_scope == 0 else -1
    if cfg.norm == 0:
        mu = x.mean(axis=axis, keepdims=True)
        var = ((x - mu) ** 2).mean(axis=axis, keepdims=True)
        return scale * (x - mu) / np.sqrt(var + np.float64(np.float32(cfg.layer_norm_eps))) + bias
    ms = (x ** 2).mean(axis=axis, keepdims=True)
    return scale * x / np.sqrt(ms + np.float64(np.float32(cfg.layer_norm_eps)))


def gelu(x):
    return 0.5 * x * (1.0 + np.tanh(np.float64(np.float32(0.7978845608028654)) * x *
                                    (1.0 + np.float64(np.float32(0.044715)) * x * x)))


def forward_all(cfg, params, ids, kv_round=None):
    """Returns logits for every row, float64 [S, V]."""
    p = np.asarray(params, dtype=np.float64)
    H, I, V = cfg.hidden_dim, cfg.intermediate_dim, cfg.vocab_size
    h_n, d = cfg.num_heads, head_dim(cfg)
    inner = h_n * d
    first, stride, rel = offsets(cfg)
    S = len(ids)
    ids = np.asarray(ids, dtype=np.int64)
    x = p[:V * H].reshape(V, H)[ids] + pe_table(S, H)
    causal = np.tril(np.ones((S, S), dtype=bool))
    for l in range(cfg.num_layers):
        base = first + l * stride

        def g(name, shape=None):
            o, sz = rel[name]
            a = p[base + o: base + o + sz]
            return a.reshape(shape) if shape else a

        n1 = norm(cfg, x, g("ln1_s"), g("ln1_b"))
        q = n1 @ g("wq", (H, inner))
        k = n1 @ g("wk", (H, inner))
        v = n1 @ g("wv", (H, inner))
        if cfg.use_bias:
            q, k, v = q + g("bq"), k + g("bk"), v + g("bv")
        if kv_round is not None:
            k, v = kv_round(k), kv_round(v)
        qh = q.reshape(S, h_n, d).transpose(1, 0, 2)
        kh = k.reshape(S, h_n, d).transpose(1, 0, 2)
        vh = v.reshape(S, h_n, d).transpose(1, 0, 2)
        sc = np.einsum("hid,hjd->hij", qh, kh) / np.sqrt(np.float64(d))
        sc = np.where(causal[None], sc, -np.inf)
        sc = sc - sc.max(axis=-1, keepdims=True)
        pr = np.exp(sc)
        pr /= pr.sum(axis=-1, keepdims=True)
        a = np.einsum("hij,hjd->hid", pr, vh).transpose(1, 0, 2).reshape(S, inner)
        o = a @ g("wo", (inner, H))
        if cfg.use_bias:
            o = o + g("bo")
        x = x + o
        n2 = norm(cfg, x, g("ln2_s"), g("ln2_b"))
        up = n2 @ g("w_up", (H, I))
        if cfg.use_bias:
            up = up + g("b_up")
        if cfg.activation == 0:
            act = gelu(up)
        else:
            gate = n2 @ g("w_gate", (H, I))
            if cfg.use_bias:
                gate = gate + g("b_gate")
            act = gate / (1.0 + np.exp(-gate)) * up
        dn = act @ g("w_down", (I, H))
        if cfg.use_bias:
            dn = dn + g("b_down")
        x = x + dn
    fo = first + cfg.num_layers * stride
    xf = norm(cfg, x, p[fo:fo + H], p[fo + H:fo + 2 * H])
    return xf @ p[fo + 2 * H: fo + 2 * H + H * V].reshape(H, V)
