// Host side of libcoeus_mi355x.so that drives the device: model construction (upload / conversion
// of the flat f32 parameter buffer), the stateless forward pass (ForwardModel::forward,
// MT:791-919) and KV-cache sessions.  Configuration, parameter layout and errors are in host.hip.
#include "model.hpp"

#include <cmath>

namespace coeus {

// ---------------------------------------------------------------- device buffers
int DeviceBuf::ensure(uint64_t want) {
    if (want <= bytes) return COEUS_OK;
    if (p) { (void)hipFree(p); p = nullptr; bytes = 0; }
    COEUS_HIP(hipMalloc(&p, want));
    bytes = want;
    return COEUS_OK;
}
void DeviceBuf::release() {
    if (p) (void)hipFree(p);
    p = nullptr;
    bytes = 0;
}

static uint64_t kv_elem_size(uint32_t kv_dtype) { return kv_dtype == COEUS_KV_F32 ? 4 : 2; }

int Workspace::ensure(const Model &m, uint64_t rows_needed, uint64_t logit_rows) {
    const coeus_config &c = m.cfg;
    const uint64_t H = c.hidden_dim, I = c.intermediate_dim, inner = m.L.inner_dim;
    if (rows_needed > rows) {
        COEUS_TRY(h.ensure(rows_needed * H * 4));
        COEUS_TRY(x.ensure(rows_needed * H * 4));
        COEUS_TRY(qkv.ensure(rows_needed * 3 * inner * 4));
        COEUS_TRY(att.ensure(rows_needed * inner * 4));
        COEUS_TRY(ff.ensure(rows_needed * I * 4));
        COEUS_TRY(ids.ensure(rows_needed * 8));
        COEUS_TRY(norm_part.ensure(norm_sequence_scratch_bytes()));
        if (c.weight_dtype != COEUS_W_F32) {
            uint64_t kmax = H > I ? H : I;
            if (inner > kmax) kmax = inner;
            COEUS_TRY(a_lp.ensure(rows_needed * gemm_ld(kmax) * 2));
            COEUS_TRY(b_lp.ensure(rows_needed * gemm_ld(kmax) * 2));
        }
        rows = rows_needed;
    }
    if (c.weight_dtype >= COEUS_W_Q8_0 && !w_lp.p) {
        // [n] rows of gemm_ld(k) elements for the largest weight
        uint64_t big = 3 * inner * gemm_ld(H);
        const uint64_t up = (c.activation == COEUS_ACT_SILU_GATED ? 2 : 1) * I * gemm_ld(H);
        if (up > big) big = up;
        if (H * gemm_ld(I) > big) big = H * gemm_ld(I);
        if (H * gemm_ld(inner) > big) big = H * gemm_ld(inner);
        if (c.vocab_size * gemm_ld(H) > big) big = c.vocab_size * gemm_ld(H);
        COEUS_TRY(w_lp.ensure(big * 2));
    }
    if (logit_rows) COEUS_TRY(logits.ensure(logit_rows * c.vocab_size * 4));
    // partial planes of the matmuls that this many rows would split along k (short prompts)
    if (rows_needed && !m.layers.empty()) {
        const LayerWeights &lw = m.layers[0];  // every layer has the same shapes
        uint64_t part = 0;
        for (const Weight *w : {&lw.qkv, &lw.o, &lw.up, &lw.down}) {
            const uint64_t b = gemm_split_scratch_bytes(*w, rows_needed);
            if (b > part) part = b;
        }
        if (logit_rows) {
            const uint64_t b = gemm_split_scratch_bytes(m.out, logit_rows);
            if (b > part) part = b;
        }
        if (part) COEUS_TRY(gemm_part.ensure(part));
    }
    gs.partials = (float *)gemm_part.p; gs.partials_bytes = gemm_part.bytes;
    gs.a_lp = a_lp.p; gs.a_lp_bytes = a_lp.bytes;
    gs.w_lp = w_lp.p; gs.w_lp_bytes = w_lp.bytes;
    gs.expand_budget = const_cast<uint64_t *>(&m.expand_budget);  // guarded by m.mu like the stream
    return COEUS_OK;
}

void Workspace::release() {
    h.release(); x.release(); qkv.release(); att.release(); ff.release(); ids.release();
    a_lp.release(); b_lp.release(); w_lp.release(); logits.release(); xq.release(); norm_part.release();
    gemm_part.release();
    rows = 0;
}

// ---------------------------------------------------------------- model construction
Model::~Model() {
    for (auto &l : layers) { weight_free(l.qkv); weight_free(l.o); weight_free(l.up); weight_free(l.down); }
    weight_free(out);
    if (embed) (void)hipFree(embed);
    if (pe) (void)hipFree(pe);
    if (small) (void)hipFree(small);
    ws.release();
    tmp_k.release();
    tmp_v.release();
    if (stream) (void)hipStreamDestroy(stream);
}

static int check_device() {
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n == 0)
        return fail(COEUS_DEVICE_ERROR, "no HIP device visible (%s)", hipGetErrorString(e));
    return COEUS_OK;
}

// params: host pointer to the flat buffer, or nullptr for seeded synthetic weights.
int model_create(const coeus_config &cfg, const float *params, uint64_t n_params, uint64_t seed,
                 Model **out) {
    COEUS_TRY(validate_config(cfg));
    const Layout L = make_layout(cfg);
    if (params && n_params < L.used_params)
        return fail(COEUS_INVALID_INPUT,
                    "Parameter access out of range: offset %llu + size %llu > %llu",  // MT:663-668
                    (unsigned long long)L.output_proj_offset,
                    (unsigned long long)L.output_proj_size, (unsigned long long)n_params);
    COEUS_TRY(check_device());
    std::unique_ptr<Model> m(new Model());
    m->cfg = cfg;
    if (m->cfg.max_batch == 0) m->cfg.max_batch = 1;
    m->L = L;
    m->n_params = params ? n_params : L.total_params;
    COEUS_HIP(hipStreamCreateWithFlags(&m->stream, hipStreamNonBlocking));
    hipStream_t st = m->stream;
    const uint64_t H = cfg.hidden_dim, I = cfg.intermediate_dim, V = cfg.vocab_size,
                   inner = L.inner_dim;
    const bool gated = cfg.activation == COEUS_ACT_SILU_GATED, bias = cfg.use_bias != 0;
    const uint32_t wd = cfg.weight_dtype;

    // the flat buffer goes to the device once; every weight is converted there
    float *dev_params = nullptr;
    struct Guard { float *&p; ~Guard() { if (p) (void)hipFree(p); } } guard{dev_params};
    if (params) {
        COEUS_HIP(hipMalloc((void **)&dev_params, L.used_params * 4));
        COEUS_HIP(hipMemcpy(dev_params, params, L.used_params * 4, hipMemcpyHostToDevice));
    }
    auto value = [&](uint64_t idx, float mean) -> float {
        if (params) return params[idx];
        const float z = synth_value_host(seed, idx);
        return mean != 0.0f ? mean + z : z;
    };

    // ---- small parameters (norm scales/biases, linear biases), assembled on the host
    const uint64_t up_rows = gated ? 2 * I : I;
    const uint64_t per_layer = 2 * H + 3 * inner + H + 2 * H + up_rows + H;
    std::vector<float> sm(cfg.num_layers * per_layer + 2 * H, 0.0f);
    for (uint64_t l = 0; l < cfg.num_layers; l++) {
        const uint64_t base = L.first_layer_offset + l * L.layer_stride;
        float *d = sm.data() + l * per_layer;
        for (uint64_t i = 0; i < H; i++) d[i] = value(base + L.ln1_scale + i, 1.0f);
        for (uint64_t i = 0; i < H; i++) d[H + i] = value(base + L.ln1_bias + i, 0.0f);
        float *bqkv = d + 2 * H, *bo = bqkv + 3 * inner, *ln2 = bo + H, *bup = ln2 + 2 * H,
              *bdown = bup + up_rows;
        for (uint64_t i = 0; i < H; i++) ln2[i] = value(base + L.ln2_scale + i, 1.0f);
        for (uint64_t i = 0; i < H; i++) ln2[H + i] = value(base + L.ln2_bias + i, 0.0f);
        if (bias) {
            for (uint64_t i = 0; i < inner; i++) {
                bqkv[i] = value(base + L.bq + i, 0.0f);
                bqkv[inner + i] = value(base + L.bk + i, 0.0f);
                bqkv[2 * inner + i] = value(base + L.bv + i, 0.0f);
            }
            for (uint64_t i = 0; i < H; i++) bo[i] = value(base + L.bo + i, 0.0f);
            for (uint64_t i = 0; i < I; i++) {
                if (gated) {
                    bup[2 * i] = value(base + L.b_gate + i, 0.0f);
                    bup[2 * i + 1] = value(base + L.b_up + i, 0.0f);
                } else {
                    bup[i] = value(base + L.b_up + i, 0.0f);
                }
            }
            for (uint64_t i = 0; i < H; i++) bdown[i] = value(base + L.b_down + i, 0.0f);
        }
    }
    {
        float *d = sm.data() + cfg.num_layers * per_layer;
        for (uint64_t i = 0; i < H; i++) d[i] = value(L.final_ln_offset + i, 1.0f);
        for (uint64_t i = 0; i < H; i++) d[H + i] = value(L.final_ln_offset + H + i, 0.0f);
    }
    COEUS_HIP(hipMalloc((void **)&m->small, sm.size() * 4));
    COEUS_HIP(hipMemcpy(m->small, sm.data(), sm.size() * 4, hipMemcpyHostToDevice));
    m->weight_bytes += sm.size() * 4;

    // ---- linear weights
    m->layers.resize(cfg.num_layers);
    for (uint64_t l = 0; l < cfg.num_layers; l++) {
        const uint64_t base = L.first_layer_offset + l * L.layer_stride;
        LayerWeights &lw = m->layers[l];
        const float *d = m->small + l * per_layer;
        lw.ln1_s = d; lw.ln1_b = d + H;
        lw.b_qkv = bias ? d + 2 * H : nullptr;
        lw.b_o = bias ? d + 2 * H + 3 * inner : nullptr;
        lw.ln2_s = d + 2 * H + 3 * inner + H; lw.ln2_b = lw.ln2_s + H;
        lw.b_up = bias ? lw.ln2_b + H : nullptr;
        lw.b_down = bias ? lw.ln2_b + H + up_rows : nullptr;
        WeightSource src;
        src.params = dev_params;
        src.seed = seed;
        // Wq | Wk | Wv are consecutive [H, inner] matrices (MT:180-182): one fused matmul
        COEUS_TRY(weight_alloc(lw.qkv, wd, H, 3 * inner));
        src.base = base + L.wq; src.n_part = inner; src.interleave = 0;
        COEUS_TRY(weight_pack(lw.qkv, src, st));
        COEUS_TRY(weight_alloc(lw.o, wd, inner, H));
        src.base = base + L.wo; src.n_part = H;
        COEUS_TRY(weight_pack(lw.o, src, st));
        COEUS_TRY(weight_alloc(lw.up, wd, H, up_rows));
        if (gated) { src.base = base + L.w_gate; src.n_part = I; src.interleave = 1; }
        else { src.base = base + L.w_up; src.n_part = I; src.interleave = 0; }
        COEUS_TRY(weight_pack(lw.up, src, st));
        COEUS_TRY(weight_alloc(lw.down, wd, I, H));
        src.base = base + L.w_down; src.n_part = H; src.interleave = 0;
        COEUS_TRY(weight_pack(lw.down, src, st));
        m->weight_bytes += lw.qkv.bytes + lw.o.bytes + lw.up.bytes + lw.down.bytes;
        // resident f16 copies for the prompt pass, while the budget lasts
        for (const Weight *w : {&lw.qkv, &lw.o, &lw.up, &lw.down}) COEUS_TRY(weight_expand(*w, &m->expand_budget, st));
    }
    m->fin_s = m->small + cfg.num_layers * per_layer;
    m->fin_b = m->fin_s + H;
    {
        WeightSource src;
        src.params = dev_params; src.seed = seed;
        src.base = L.output_proj_offset; src.n_part = V;
        COEUS_TRY(weight_alloc(m->out, wd, H, V));
        COEUS_TRY(weight_pack(m->out, src, st));
        m->weight_bytes += m->out.bytes;
    }

    // ---- token embedding: bf16 with bf16 weights, f32 otherwise
    m->embed_bf16 = wd == COEUS_W_BF16;
    {
        const uint64_t n = V * H;
        float *src32 = dev_params;  // embedding sits at offset 0
        float *tmp = nullptr;
        if (!params) {
            COEUS_HIP(hipMalloc((void **)&tmp, n * 4));
            int rc = launch_fill_seeded(tmp, n, seed, 0, 0.0f, st);
            if (rc != COEUS_OK) { (void)hipFree(tmp); return rc; }
            src32 = tmp;
        }
        if (m->embed_bf16) {
            hipError_t e = hipMalloc(&m->embed, n * 2);
            int rc = e == hipSuccess ? launch_f32_to_bf16(src32, (uint16_t *)m->embed, n, st)
                                     : fail(COEUS_OUT_OF_MEMORY, "hipMalloc(embedding) failed");
            hipError_t e2 = hipStreamSynchronize(st);
            if (tmp) (void)hipFree(tmp);
            if (rc != COEUS_OK) return rc;
            COEUS_HIP(e2);
            m->weight_bytes += n * 2;
        } else if (tmp) {
            m->embed = tmp;  // keep the generated table
            m->weight_bytes += n * 4;
        } else {
            COEUS_HIP(hipMalloc(&m->embed, n * 4));
            COEUS_HIP(hipMemcpyAsync(m->embed, src32, n * 4, hipMemcpyDeviceToDevice, st));
            m->weight_bytes += n * 4;
        }
    }

    // ---- sinusoidal table (MT:398-407), computed with the host libm and uploaded
    {
        std::vector<float> t(cfg.max_seq_len * H);
        positional_encoding_host(cfg.max_seq_len, H, t.data());
        COEUS_HIP(hipMalloc((void **)&m->pe, t.size() * 4));
        COEUS_HIP(hipMemcpy(m->pe, t.data(), t.size() * 4, hipMemcpyHostToDevice));
    }
    COEUS_HIP(hipStreamSynchronize(st));
    *out = m.release();
    return COEUS_OK;
}

// ---------------------------------------------------------------- forward over rows (prefill path)
// Runs embedding + all blocks for `batch` sequences of n new rows each (positions pos0..),
// appending K/V to `cache`; leaves the residual stream in ws.h.  Uses the matrix-core matmul.
int run_blocks_prefill(Model &m, Workspace &ws, const Cache &cache, uint64_t batch, uint64_t n,
                       uint64_t pos0, hipStream_t st) {
    const coeus_config &c = m.cfg;
    const uint64_t H = c.hidden_dim, rows = batch * n, hd = m.L.head_dim;
    float *h = (float *)ws.h.p, *x = (float *)ws.x.p, *qkv = (float *)ws.qkv.p,
          *att = (float *)ws.att.p, *ff = (float *)ws.ff.p;
    COEUS_TRY(launch_embed(m.embed, m.embed_bf16, m.pe, (const uint64_t *)ws.ids.p, rows, n, pos0,
                           nullptr, H, h, nullptr, st));
    // With 16-bit matrix-core operands the producers write the next matmul's A operand directly
    // (norm -> a_lp, attention -> b_lp, FFN-up epilogue -> b_lp) instead of an f32 buffer that a
    // conversion pass would read back.  Needs per-token norms (the whole-sequence norm is the
    // reference-parity mode and stays on the f32 route).
    const bool lp = c.weight_dtype != COEUS_W_F32 && c.norm_scope == COEUS_SCOPE_TOKEN && ws.a_lp.p && ws.b_lp.p;
    const bool lp_bf = c.weight_dtype == COEUS_W_BF16;
    const bool attn_lp = lp && attn_prefill_on_matrix_cores(n, hd, c.kv_dtype);
    const LpOut x_lp{ws.a_lp.p, gemm_ld(H), lp_bf};
    const LpOut att_lp{ws.b_lp.p, gemm_ld(m.L.inner_dim), lp_bf};
    const LpOut ff_lp{ws.b_lp.p, gemm_ld(c.intermediate_dim), lp_bf};
    for (uint64_t l = 0; l < c.num_layers; l++) {
        const LayerWeights &lw = m.layers[l];
        char *kc = (char *)cache.k + (cache.per_layer ? l * cache.layer_bytes : 0);
        char *vc = (char *)cache.v + (cache.per_layer ? l * cache.layer_bytes : 0);
        // h -> LN1 -> q|k|v (MT:469, MT:185-214)
        COEUS_TRY(launch_norm(c.norm, c.norm_scope, h, rows, H, lw.ln1_s, lw.ln1_b, c.layer_norm_eps,
                              lp ? nullptr : x, nullptr, 0, st, lp ? &x_lp : nullptr, (double *)ws.norm_part.p));
        Epilogue e1;
        e1.bias = lw.b_qkv; e1.out_f32 = qkv;
        // the matrix-core matmul writes the key and value thirds straight into the cache
        const bool fused_append = gemm_appends_kv(lw.qkv, rows, m.L.inner_dim, hd);
        if (fused_append) {
            e1.kv_k = kc; e1.kv_v = vc; e1.kv_dtype = c.kv_dtype;
            e1.kv_inner = (uint32_t)m.L.inner_dim; e1.kv_heads = (uint32_t)c.num_heads;
            e1.kv_hd = (uint32_t)hd; e1.kv_max_ctx = (uint32_t)cache.max_ctx;
            e1.kv_rows_per_seq = (uint32_t)n; e1.kv_pos0 = (uint32_t)pos0;
        }
        COEUS_TRY(launch_gemm(lw.qkv, lp ? (const void *)ws.a_lp.p : (const void *)x, rows, e1, ws.gs, st, lp));
        if (!fused_append)
            COEUS_TRY(launch_kv_append(qkv, kc, vc, c.kv_dtype, batch, n, c.num_heads, hd, cache.max_ctx,
                                       pos0, nullptr, st));
        COEUS_TRY(launch_attention(qkv, kc, vc, c.kv_dtype, batch, n, c.num_heads, hd, cache.max_ctx,
                                   pos0, nullptr, attn_lp ? nullptr : att, nullptr, 0, nullptr, 0, nullptr,
                                   st, attn_lp ? &att_lp : nullptr));
        // output projection + bias + residual (MT:281-299, MT:481-485)
        Epilogue e2;
        e2.bias = lw.b_o; e2.residual = h; e2.out_f32 = h;
        COEUS_TRY(launch_gemm(lw.o, attn_lp ? (const void *)ws.b_lp.p : (const void *)att, rows, e2, ws.gs, st, attn_lp));
        // LN2 -> FFN -> residual (MT:488-496, MT:339-375)
        COEUS_TRY(launch_norm(c.norm, c.norm_scope, h, rows, H, lw.ln2_s, lw.ln2_b, c.layer_norm_eps,
                              lp ? nullptr : x, nullptr, 0, st, lp ? &x_lp : nullptr, (double *)ws.norm_part.p));
        Epilogue e3;
        e3.bias = lw.b_up;
        if (lp) e3.out_lp = ff_lp; else e3.out_f32 = ff;
        e3.act = c.activation == COEUS_ACT_SILU_GATED ? COEUS_EPI_SILU_GATE : COEUS_EPI_GELU;
        COEUS_TRY(launch_gemm(lw.up, lp ? (const void *)ws.a_lp.p : (const void *)x, rows, e3, ws.gs, st, lp));
        Epilogue e4;
        e4.bias = lw.b_down; e4.residual = h; e4.out_f32 = h;
        COEUS_TRY(launch_gemm(lw.down, lp ? (const void *)ws.b_lp.p : (const void *)ff, rows, e4, ws.gs, st, lp));
    }
    return COEUS_OK;
}

// Logits of `count` contiguous rows of x (already normalised) through the decode matmul.
static int logits_gemv(Model &m, Workspace &ws, const float *x_rows, uint64_t count, float *logits,
                       hipStream_t st) {
    for (uint64_t r0 = 0; r0 < count; r0 += 16) {
        const uint64_t b = count - r0 < 16 ? count - r0 : 16;
        Epilogue e;
        e.out_f32 = logits + r0 * m.cfg.vocab_size;
        const void *xin = x_rows + r0 * m.cfg.hidden_dim;
        if (m.out.dtype >= COEUS_W_Q8_0) {
            COEUS_TRY(ws.xq.ensure(m.out.k_pad * 16 * 2));
            COEUS_TRY(launch_pack_xq(x_rows + r0 * m.cfg.hidden_dim, b, m.out.k, m.out.k_pad,
                                     (__half *)ws.xq.p, st));
            xin = ws.xq.p;
        }
        COEUS_TRY(launch_gemv(m.out, xin, b, e, st));
    }
    return COEUS_OK;
}

static int check_ids(const Model &m, const uint64_t *ids, uint64_t count) {
    const uint64_t V = m.cfg.vocab_size;
    for (uint64_t i = 0; i < count; i++)
        if (ids[i] >= V)  // MT:816-822
            return fail(COEUS_INVALID_INPUT, "Token ID %llu out of range [0, %llu]",
                        (unsigned long long)ids[i], (unsigned long long)(V - 1));
    return COEUS_OK;
}

int model_forward(Model &m, const uint64_t *ids, uint64_t seq_len, float *logits_out, bool all_rows) {
    const coeus_config &c = m.cfg;
    if (!ids || !logits_out) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    if (seq_len == 0 || seq_len > c.max_seq_len)  // MT:797-802 (empty input panics there, MT:915)
        return fail(COEUS_INVALID_INPUT, "Sequence length %llu out of range [1, %llu]",
                    (unsigned long long)seq_len, (unsigned long long)c.max_seq_len);
    COEUS_TRY(check_ids(m, ids, seq_len));
    std::lock_guard<std::mutex> lock(m.mu);
    hipStream_t st = m.stream;
    const uint64_t H = c.hidden_dim, V = c.vocab_size;
    COEUS_TRY(m.ws.ensure(m, seq_len, all_rows ? seq_len : 1));
    // single-layer scratch cache: the stateless forward needs K/V only inside a layer
    const uint64_t cache_bytes = c.num_heads * seq_len * m.L.head_dim * kv_elem_size(c.kv_dtype);
    COEUS_TRY(m.tmp_k.ensure(cache_bytes));
    COEUS_TRY(m.tmp_v.ensure(cache_bytes));
    Cache cache{m.tmp_k.p, m.tmp_v.p, seq_len, 0, false};
    COEUS_HIP(hipMemcpyAsync(m.ws.ids.p, ids, seq_len * 8, hipMemcpyHostToDevice, st));
    COEUS_TRY(run_blocks_prefill(m, m.ws, cache, 1, seq_len, 0, st));
    float *h = (float *)m.ws.h.p, *x = (float *)m.ws.x.p, *logits = (float *)m.ws.logits.p;
    // final normalisation over the whole slice, then the last row (MT:903-916) or every row
    COEUS_TRY(launch_norm(c.norm, c.norm_scope, h, seq_len, H, m.fin_s, m.fin_b, c.layer_norm_eps, x,
                          nullptr, 0, st, nullptr, (double *)m.ws.norm_part.p));
    if (all_rows) {
        Epilogue e;
        e.out_f32 = logits;
        COEUS_TRY(launch_gemm(m.out, x, seq_len, e, m.ws.gs, st));
    } else {
        COEUS_TRY(logits_gemv(m, m.ws, x + (seq_len - 1) * H, 1, logits, st));
    }
    COEUS_HIP(hipMemcpyAsync(logits_out, logits, (all_rows ? seq_len : 1) * V * 4,
                             hipMemcpyDeviceToHost, st));
    COEUS_HIP(hipStreamSynchronize(st));
    return COEUS_OK;
}

// ---------------------------------------------------------------- sessions
Session::~Session() {
    if (graph_exec) (void)hipGraphExecDestroy(graph_exec);
    if (graph) (void)hipGraphDestroy(graph);
    kc.release(); vc.release(); ws.release();
    dh.release(); dx.release(); dqkv.release(); datt.release(); dff.release(); dlogits.release();
    dids.release(); dpos.release(); dhist.release(); dpart.release(); dcount.release(); dstats.release();
    xq_h.release(); xq_inner.release(); xq_ff.release(); xq_g.release();
}

int session_create(Model &m, uint64_t batch, uint64_t max_ctx, Session **out) {
    const coeus_config &c = m.cfg;
    if (c.norm_scope != COEUS_SCOPE_TOKEN)
        return fail(COEUS_INVALID_CONFIG,
                    "Invalid configuration: norm_scope = 0: a KV cache needs per-token "
                    "normalisation (whole-sequence statistics change cached rows)");
    if (batch == 0 || batch > c.max_batch)
        return fail(COEUS_INVALID_INPUT, "Batch %llu out of range [1, %llu]",
                    (unsigned long long)batch, (unsigned long long)c.max_batch);
    if (max_ctx == 0 || max_ctx > c.max_seq_len)
        return fail(COEUS_INVALID_INPUT, "Sequence length %llu out of range [1, %llu]",
                    (unsigned long long)max_ctx, (unsigned long long)c.max_seq_len);
    std::unique_ptr<Session> s(new Session());
    s->m = &m;
    s->batch = batch;
    s->max_ctx = max_ctx;
    s->use_graph = graph_replay_forbidden() == nullptr;
    const uint64_t H = c.hidden_dim, I = c.intermediate_dim, V = c.vocab_size,
                   inner = m.L.inner_dim, hd = m.L.head_dim;
    s->layer_bytes = batch * c.num_heads * max_ctx * hd * kv_elem_size(c.kv_dtype);
    COEUS_TRY(s->kc.ensure(s->layer_bytes * c.num_layers));
    COEUS_TRY(s->vc.ensure(s->layer_bytes * c.num_layers));
    // decode-step buffers
    COEUS_TRY(s->dh.ensure(batch * H * 4));
    COEUS_TRY(s->dx.ensure(batch * H * 4));
    COEUS_TRY(s->dqkv.ensure(batch * 3 * inner * 4));
    COEUS_TRY(s->datt.ensure(batch * inner * 4));
    COEUS_TRY(s->dff.ensure(batch * I * 4));
    COEUS_TRY(s->dlogits.ensure(batch * V * 4));
    COEUS_TRY(s->dids.ensure(batch * 8));
    COEUS_TRY(s->dpos.ensure(64));
    COEUS_TRY(s->dhist.ensure(batch * max_ctx * 8));
    s->nsplit = attn_decode_splits(batch, c.num_heads, max_ctx);
    COEUS_TRY(s->dpart.ensure(batch * c.num_heads * s->nsplit * (hd + 2) * 4));
    COEUS_TRY(s->dcount.ensure(batch * c.num_heads * 4));
    COEUS_HIP(hipMemset(s->dcount.p, 0, s->dcount.bytes));
    COEUS_TRY(s->dstats.ensure(batch * ceil_div(c.hidden_dim, 16) * sizeof(float2)));
    COEUS_HIP(hipMemset(s->dstats.p, 0, s->dstats.bytes));
    s->bp = pad_batch(batch);
    if (c.weight_dtype >= COEUS_W_Q8_0) {
        // f16 activation buffers in the decode matmul's interchange format; padding stays zero
        COEUS_TRY(s->xq_h.ensure(round_up(H, 128) * s->bp * 2));
        COEUS_TRY(s->xq_inner.ensure(round_up(inner, 128) * s->bp * 2));
        COEUS_TRY(s->xq_ff.ensure(round_up(I, 128) * s->bp * 2));
        COEUS_HIP(hipMemset(s->xq_h.p, 0, s->xq_h.bytes));
        COEUS_HIP(hipMemset(s->xq_inner.p, 0, s->xq_inner.bytes));
        COEUS_HIP(hipMemset(s->xq_ff.p, 0, s->xq_ff.bytes));
        // the residual rows times the next root-mean-square norm's scale (NormFuse::g)
        COEUS_TRY(s->xq_g.ensure(batch * H * 4));
        COEUS_HIP(hipMemset(s->xq_g.p, 0, s->xq_g.bytes));
    }
    *out = s.release();
    return COEUS_OK;
}

int session_prefill(Session &s, const uint64_t *ids, uint64_t n, float *logits_out) {
    Model &m = *s.m;
    const coeus_config &c = m.cfg;
    if (!ids) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    // the position is read and advanced under the lock: two threads stepping one session must not
    // both pass the bound below and then write a cache row past the end
    std::lock_guard<std::mutex> lock(m.mu);
    if (n == 0 || n > s.max_ctx || s.pos + n > s.max_ctx)
        return fail(COEUS_INVALID_INPUT, "Sequence length %llu out of range [1, %llu]",
                    (unsigned long long)(s.pos + n), (unsigned long long)s.max_ctx);
    COEUS_TRY(check_ids(m, ids, s.batch * n));
    hipStream_t st = m.stream;
    const uint64_t H = c.hidden_dim, V = c.vocab_size, rows = s.batch * n;
    COEUS_TRY(s.ws.ensure(m, rows, 0));
    Cache cache{s.kc.p, s.vc.p, s.max_ctx, s.layer_bytes, true};
    COEUS_HIP(hipMemcpyAsync(s.ws.ids.p, ids, rows * 8, hipMemcpyHostToDevice, st));
    COEUS_TRY(run_blocks_prefill(m, s.ws, cache, s.batch, n, s.pos, st));
    s.pos += n;
    if (logits_out) {
        // last row of every sequence -> contiguous [batch, H], final norm, decode matmul
        float *h = (float *)s.ws.h.p, *last = (float *)s.dh.p, *x = (float *)s.dx.p;
        COEUS_HIP(hipMemcpy2DAsync(last, H * 4, h + (n - 1) * H, n * H * 4, H * 4, s.batch,
                                   hipMemcpyDeviceToDevice, st));
        COEUS_TRY(launch_norm(c.norm, COEUS_SCOPE_TOKEN, last, s.batch, H, m.fin_s, m.fin_b,
                              c.layer_norm_eps, x, nullptr, 0, st));
        COEUS_TRY(logits_gemv(m, s.ws, x, s.batch, (float *)s.dlogits.p, st));
        COEUS_HIP(hipMemcpyAsync(logits_out, s.dlogits.p, s.batch * V * 4, hipMemcpyDeviceToHost, st));
    }
    COEUS_HIP(hipStreamSynchronize(st));
    return COEUS_OK;
}

// One decode step for every sequence of the session, reading the token ids from s.dids and the
// position from the device (s.dpos[0]); only enqueues kernels, so it can be graph-captured.
static uint64_t gemv_algorithmic_bytes(const Weight &w, uint64_t batch, bool gated, bool normed);

// `only` (roofline measurements): enqueue just the decode matmuls (with their fused staging and
// epilogues) or just the attention launches, and count them and their algorithmic bytes.
enum { STEP_ALL = 0, STEP_MATMULS = 1, STEP_ATTENTION = 2 };
static int enqueue_decode_step(Session &s, hipStream_t st, int only = STEP_ALL,
                               uint64_t *launches = nullptr, uint64_t *bytes = nullptr) {
    const bool matmuls_only = only != STEP_ALL;  // everything that is not a matmul or the attention is skipped
    const bool with_matmuls = only != STEP_ATTENTION, with_attention = only != STEP_MATMULS;
    Model &m = *s.m;
    const coeus_config &c = m.cfg;
    const uint64_t H = c.hidden_dim, B = s.batch, hd = m.L.head_dim;
    const bool quant = c.weight_dtype >= COEUS_W_Q8_0;
    const uint32_t bp = s.bp;
    const uint32_t *pos_dev = (const uint32_t *)s.dpos.p;
    float *h = (float *)s.dh.p, *x = (float *)s.dx.p, *qkv = (float *)s.dqkv.p,
          *att = (float *)s.datt.p, *ff = (float *)s.dff.p;
    __half *xq_h = (__half *)s.xq_h.p, *xq_inner = (__half *)s.xq_inner.p, *xq_ff = (__half *)s.xq_ff.p;
    // Producers of the residual stream h (embedding, Wo and FFN-down epilogues) also write
    // per-16-element {sum, M2} records of it; the matmul that follows merges them into the row
    // statistics of its folded norm.
    float2 *stats = (quant && s.fuse) ? (float2 *)s.dstats.p : nullptr;
    // Root-mean-square norms folded into the next matmul: the producers of h also store
    // h * scale of the norm that follows (Epilogue::g_out), which is what that matmul stages.
    const bool gpath = stats && c.norm == COEUS_NORM_RMSNORM && gemv_can_fuse_norm(m.layers[0].qkv, B) &&
                       gemv_can_fuse_norm(m.layers[0].up, B) && gemv_can_fuse_norm(m.out, B);
    float *xq_g = gpath ? (float *)s.xq_g.p : nullptr;
    if (!matmuls_only)
        COEUS_TRY(launch_embed(m.embed, m.embed_bf16, m.pe, (const uint64_t *)s.dids.p, B, 1, 0,
                               pos_dev, H, h, stats, st, gpath ? m.layers[0].ln1_s : nullptr, xq_g));
    uint64_t n_launch = 0, n_bytes = 0;
    const bool gated_ffn = c.activation == COEUS_ACT_SILU_GATED;
    // Per layer: [norm1 -> q|k|v (+ cache append)] -> attention (+ merge) -> [Wo + residual] ->
    // [norm2 -> FFN up (+ activation)] -> [FFN down + residual].  With quantised weights whose
    // activation block fits in LDS the norms run inside the matmul's staging: 5 launches a layer.
    auto normed_gemv = [&](const Weight &w, const float *ns, const float *nb, const Epilogue &e) -> int {
        if (!with_matmuls) return COEUS_OK;
        n_launch++;
        if (quant && s.fuse && gemv_can_fuse_norm(w, B)) {
            NormFuse nf;
            nf.h = h; nf.scale = ns; nf.bias = nb; nf.eps = c.layer_norm_eps; nf.kind = c.norm;
            nf.stats = stats;
            nf.g = xq_g;
            n_bytes += gemv_algorithmic_bytes(w, B, e.act == COEUS_EPI_SILU_GATE, true);
            return launch_gemv(w, nullptr, B, e, st, &nf);
        }
        // (dense weights: every workgroup of 16 output rows normalises the activation rows for
        // itself, which pays for a few hundred workgroups but not for the 3142 of a 50257-row logits
        // projection: 30 us folded against 4 + 19 us as two launches on the 250M bf16 model)
        if (!quant && s.fuse && gemv_can_fuse_norm_dense(w, B) && w.n <= 16384) {
            NormFuse nf;
            nf.h = h; nf.scale = ns; nf.bias = nb; nf.eps = c.layer_norm_eps; nf.kind = c.norm;
            n_bytes += gemv_algorithmic_bytes(w, B, e.act == COEUS_EPI_SILU_GATE, true);
            return launch_gemv(w, nullptr, B, e, st, &nf);
        }
        n_bytes += gemv_algorithmic_bytes(w, B, e.act == COEUS_EPI_SILU_GATE, false);
        if (!matmuls_only) {
            if (stats && (H & 7) == 0) {  // row statistics from the producer's records
                NormFuse nf;
                nf.h = h; nf.scale = ns; nf.bias = nb; nf.eps = c.layer_norm_eps; nf.kind = c.norm;
                nf.stats = stats;
                COEUS_TRY(launch_norm_from_stats(nf, B, H, w.k_pad, xq_h, st));
            } else {
                COEUS_TRY(launch_norm(c.norm, COEUS_SCOPE_TOKEN, h, B, H, ns, nb, c.layer_norm_eps,
                                      quant ? nullptr : x, quant ? xq_h : nullptr, bp, st));
            }
        }
        return launch_gemv(w, quant ? (const void *)xq_h : (const void *)x, B, e, st);
    };
    auto plain_gemv = [&](const Weight &w, const void *xin, const Epilogue &e) -> int {
        if (!with_matmuls) return COEUS_OK;
        n_launch++;
        n_bytes += gemv_algorithmic_bytes(w, B, false, false) + (e.g_out ? B * w.n * 4 : 0);
        return launch_gemv(w, xin, B, e, st);
    };
    for (uint64_t l = 0; l < c.num_layers; l++) {
        const LayerWeights &lw = m.layers[l];
        char *kc = (char *)s.kc.p + l * s.layer_bytes, *vc = (char *)s.vc.p + l * s.layer_bytes;
        Epilogue e1;
        e1.bias = lw.b_qkv; e1.out_f32 = qkv;
        e1.kv_k = kc; e1.kv_v = vc; e1.kv_pos = pos_dev; e1.kv_dtype = c.kv_dtype;
        e1.kv_inner = (uint32_t)m.L.inner_dim; e1.kv_heads = (uint32_t)c.num_heads;
        e1.kv_hd = (uint32_t)hd; e1.kv_max_ctx = (uint32_t)s.max_ctx;
        COEUS_TRY(normed_gemv(lw.qkv, lw.ln1_s, lw.ln1_b, e1));
        if (with_attention) {
            COEUS_TRY(launch_attention(qkv, kc, vc, c.kv_dtype, B, 1, c.num_heads, hd, s.max_ctx, 0,
                                       pos_dev, quant ? nullptr : att, quant ? xq_inner : nullptr,
                                       bp, (float *)s.dpart.p, s.nsplit, (uint32_t *)s.dcount.p, st));
            if (only == STEP_ATTENTION) {
                // keys and values of every cached position of every (sequence, head), the query
                // and the output row; the position is read by the caller before the capture
                n_launch++;
                n_bytes += B * c.num_heads * hd * ((uint64_t)(s.host_pos[0] + 1) * 2 * kv_elem_size(c.kv_dtype) + 8);
            }
        }
        Epilogue e2;
        e2.bias = lw.b_o; e2.residual = h; e2.out_f32 = h; e2.stats_out = stats;
        if (gpath) { e2.g_scale = lw.ln2_s; e2.g_out = xq_g; }
        COEUS_TRY(plain_gemv(lw.o, quant ? (const void *)xq_inner : (const void *)att, e2));
        Epilogue e3;
        e3.bias = lw.b_up;
        e3.act = gated_ffn ? COEUS_EPI_SILU_GATE : COEUS_EPI_GELU;
        if (quant) { e3.out_xq = xq_ff; e3.bp_out = bp; } else e3.out_f32 = ff;
        COEUS_TRY(normed_gemv(lw.up, lw.ln2_s, lw.ln2_b, e3));
        Epilogue e4;
        e4.bias = lw.b_down; e4.residual = h; e4.out_f32 = h; e4.stats_out = stats;
        if (gpath) { e4.g_scale = l + 1 < c.num_layers ? m.layers[l + 1].ln1_s : m.fin_s; e4.g_out = xq_g; }
        COEUS_TRY(plain_gemv(lw.down, quant ? (const void *)xq_ff : (const void *)ff, e4));
    }
    Epilogue eo;
    eo.out_f32 = (float *)s.dlogits.p;
    COEUS_TRY(normed_gemv(m.out, m.fin_s, m.fin_b, eo));
    if (launches) *launches = n_launch;
    if (bytes) *bytes = n_bytes;
    return COEUS_OK;
}

static int upload_pos(Session &s, hipStream_t st) {
    s.host_pos[0] = (uint32_t)s.pos;
    s.host_pos[1] = 0;
    COEUS_HIP(hipMemcpyAsync(s.dpos.p, s.host_pos, 8, hipMemcpyHostToDevice, st));
    return COEUS_OK;
}

int session_decode(Session &s, const uint64_t *ids, float *logits_out) {
    Model &m = *s.m;
    if (!ids) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    std::lock_guard<std::mutex> lock(m.mu);  // before any read of the position (see session_prefill)
    if (s.pos + 1 > s.max_ctx)
        return fail(COEUS_INVALID_INPUT, "Sequence length %llu out of range [1, %llu]",
                    (unsigned long long)(s.pos + 1), (unsigned long long)s.max_ctx);
    COEUS_TRY(check_ids(m, ids, s.batch));
    hipStream_t st = m.stream;
    COEUS_HIP(hipMemcpyAsync(s.dids.p, ids, s.batch * 8, hipMemcpyHostToDevice, st));
    COEUS_TRY(upload_pos(s, st));
    COEUS_TRY(enqueue_decode_step(s, st));
    s.pos += 1;
    if (logits_out)
        COEUS_HIP(hipMemcpyAsync(logits_out, s.dlogits.p, s.batch * m.cfg.vocab_size * 4,
                                 hipMemcpyDeviceToHost, st));
    COEUS_HIP(hipStreamSynchronize(st));
    return COEUS_OK;
}

// step + argmax (feeds the next step) + position advance, captured once and replayed.
static int build_greedy_graph(Session &s, hipStream_t st) {
    Model &m = *s.m;
    COEUS_HIP(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
    int rc = enqueue_decode_step(s, st);
    // {position, step} sit next to each other in dpos; a single sequence's argmax moves them on
    const bool fold = s.batch == 1;
    if (rc == COEUS_OK)
        rc = launch_argmax((const float *)s.dlogits.p, s.batch, m.cfg.vocab_size, (uint64_t *)s.dids.p,
                           (uint64_t *)s.dhist.p, s.max_ctx, (const uint32_t *)s.dpos.p + 1, st,
                           fold ? (uint32_t *)s.dpos.p : nullptr);
    if (rc == COEUS_OK && !fold) rc = launch_advance((uint32_t *)s.dpos.p, (uint32_t *)s.dpos.p + 1, st);
    hipGraph_t g = nullptr;
    hipError_t e = hipStreamEndCapture(st, &g);
    if (rc != COEUS_OK) { if (g) (void)hipGraphDestroy(g); return rc; }
    COEUS_HIP(e);
    s.graph = g;
    COEUS_HIP(hipGraphInstantiate(&s.graph_exec, s.graph, nullptr, nullptr, 0));
    return COEUS_OK;
}

int session_decode_greedy(Session &s, const uint64_t *first_ids, uint64_t n_steps, uint64_t *out_ids,
                          const coeus_sampling *sampling) {
    Model &m = *s.m;
    if (!first_ids || !out_ids) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    std::lock_guard<std::mutex> lock(m.mu);  // before any read of the position (see session_prefill)
    if (n_steps == 0 || n_steps > s.max_ctx || s.pos + n_steps > s.max_ctx)
        return fail(COEUS_INVALID_INPUT, "Sequence length %llu out of range [1, %llu]",
                    (unsigned long long)(s.pos + n_steps), (unsigned long long)s.max_ctx);
    COEUS_TRY(check_ids(m, first_ids, s.batch));
    hipStream_t st = m.stream;
    const bool sample = sampling && sampling->temperature > 0.f;
    if (!sample && !s.graph_exec && s.use_graph) COEUS_TRY(build_greedy_graph(s, st));
    COEUS_HIP(hipMemcpyAsync(s.dids.p, first_ids, s.batch * 8, hipMemcpyHostToDevice, st));
    COEUS_TRY(upload_pos(s, st));
    for (uint64_t i = 0; i < n_steps; i++) {
        if (!sample && s.use_graph) {
            COEUS_HIP(hipGraphLaunch(s.graph_exec, st));
        } else {
            COEUS_TRY(enqueue_decode_step(s, st));
            if (sample)  // the token drawn here takes position *dpos + 1
                COEUS_TRY(launch_sample((const float *)s.dlogits.p, s.batch, m.cfg.vocab_size, *sampling, 1,
                                        (const uint32_t *)s.dpos.p, (uint64_t *)s.dids.p,
                                        (uint64_t *)s.dhist.p, s.max_ctx, (const uint32_t *)s.dpos.p + 1, st));
            else
                COEUS_TRY(launch_argmax((const float *)s.dlogits.p, s.batch, m.cfg.vocab_size,
                                        (uint64_t *)s.dids.p, (uint64_t *)s.dhist.p, s.max_ctx,
                                        (const uint32_t *)s.dpos.p + 1, st,
                                        s.batch == 1 ? (uint32_t *)s.dpos.p : nullptr));
            if (sample || s.batch != 1)
                COEUS_TRY(launch_advance((uint32_t *)s.dpos.p, (uint32_t *)s.dpos.p + 1, st));
        }
    }
    COEUS_HIP(hipMemcpy2DAsync(out_ids, n_steps * 8, s.dhist.p, s.max_ctx * 8, n_steps * 8, s.batch,
                               hipMemcpyDeviceToHost, st));
    COEUS_HIP(hipStreamSynchronize(st));
    s.pos += n_steps;
    return COEUS_OK;
}

// Algorithmic bytes one launch of the decode matmul moves: the weight in its stored form
// (quants + scales, padding excluded) plus the activation rows in (f32 when the norm is folded
// into the launch, else the matrix-core input type) and out.
static uint64_t gemv_algorithmic_bytes(const Weight &w, uint64_t batch, bool gated, bool normed) {
    uint64_t wb;
    switch (w.dtype) {
        case COEUS_W_F32: wb = w.k * w.n * 4; break;
        case COEUS_W_BF16: wb = w.k * w.n * 2; break;
        case COEUS_W_Q8_0: wb = w.k * w.n + w.k * w.n / 32 * 2; break;
        default: wb = w.k * w.n / 2 + w.k * w.n / 32 * 2; break;
    }
    const uint64_t in_b = batch * w.k * ((w.dtype >= COEUS_W_Q8_0 && !normed) ? 2 : 4);
    const uint64_t out_b = batch * (gated ? w.n / 2 : w.n) * 4;
    return wb + in_b + out_b;
}

// Replays only the decode matmuls of one step (4 per layer + the logits projection, with the
// model's real weights, shapes, fused staging and epilogues) `reps` times from a captured graph
// and times them with events on the model's stream.  The cache row at the current position and
// the decode activations are overwritten with meaningless values: reset the session afterwards.
static int session_time_decode_part(Session &s, int only, uint64_t reps, float *ms_out, uint64_t *launches_out,
                                    uint64_t *bytes_out);

int session_time_decode_matmuls(Session &s, uint64_t reps, float *ms_out, uint64_t *launches_out,
                                uint64_t *bytes_out) {
    return session_time_decode_part(s, STEP_MATMULS, reps, ms_out, launches_out, bytes_out);
}

// The same for the attention launches of one step (one per layer) at the session's current
// context length (its last cached position): the kernel that dominates a step at batch 16.
int session_time_decode_attention(Session &s, uint64_t reps, float *ms_out, uint64_t *launches_out,
                                  uint64_t *bytes_out) {
    return session_time_decode_part(s, STEP_ATTENTION, reps, ms_out, launches_out, bytes_out);
}

static int session_time_decode_part(Session &s, int only, uint64_t reps, float *ms_out, uint64_t *launches_out,
                                    uint64_t *bytes_out) {
    Model &m = *s.m;
    if (reps == 0 || !ms_out) return fail(COEUS_INVALID_INPUT, "bad timing arguments");
    std::lock_guard<std::mutex> lock(m.mu);  // before any read of the position (see session_prefill)
    if (only == STEP_ATTENTION && s.pos == 0)
        return fail(COEUS_INVALID_INPUT, "the session holds no cached position to attend to");
    hipStream_t st = m.stream;
    {   // the q|k|v epilogue writes a cache row: point it at a valid one; the attention reads
        // positions 0 .. that row, so a full session attends to its whole context
        const uint64_t keep = s.pos;
        if (s.pos >= s.max_ctx || only == STEP_ATTENTION) s.pos = (s.pos < s.max_ctx ? s.pos : s.max_ctx) - 1;
        int rc0 = upload_pos(s, st);
        s.pos = keep;
        COEUS_TRY(rc0);
    }
    uint64_t launches = 0, bytes = 0;
    auto enqueue = [&]() -> int { return enqueue_decode_step(s, st, only, &launches, &bytes); };
    if (!s.use_graph) {
        // a session switched to kernel-by-kernel launches (coeus_session_set_graph) is timed that
        // way too: profilers that cannot follow graph replays see every launch
        hipEvent_t t0 = nullptr, t1 = nullptr;
        COEUS_HIP(hipEventCreate(&t0));
        hipError_t e = hipEventCreate(&t1);
        int rc = e == hipSuccess ? enqueue() : COEUS_OK;  // untimed first pass
        if (e == hipSuccess && rc == COEUS_OK) e = hipEventRecord(t0, st);
        for (uint64_t i = 0; i < reps && e == hipSuccess && rc == COEUS_OK; i++) rc = enqueue();
        if (e == hipSuccess && rc == COEUS_OK) e = hipEventRecord(t1, st);
        if (e == hipSuccess) e = hipStreamSynchronize(st);
        float ms = 0.f;
        if (e == hipSuccess && rc == COEUS_OK) e = hipEventElapsedTime(&ms, t0, t1);
        (void)hipEventDestroy(t0);
        if (t1) (void)hipEventDestroy(t1);
        COEUS_TRY(rc);
        COEUS_HIP(e);
        *ms_out = ms;
        if (launches_out) *launches_out = launches * reps;
        if (bytes_out) *bytes_out = bytes * reps;
        return COEUS_OK;
    }
    COEUS_HIP(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
    int rc = enqueue();
    hipGraph_t g = nullptr;
    hipError_t e = hipStreamEndCapture(st, &g);
    if (rc != COEUS_OK) { if (g) (void)hipGraphDestroy(g); return rc; }
    COEUS_HIP(e);
    hipGraphExec_t ge = nullptr;
    e = hipGraphInstantiate(&ge, g, nullptr, nullptr, 0);
    if (e != hipSuccess) { (void)hipGraphDestroy(g); COEUS_HIP(e); }
    hipEvent_t t0 = nullptr, t1 = nullptr;
    (void)hipEventCreate(&t0);
    (void)hipEventCreate(&t1);
    e = hipGraphLaunch(ge, st);  // untimed first replay
    if (e == hipSuccess) e = hipEventRecord(t0, st);
    for (uint64_t i = 0; i < reps && e == hipSuccess; i++) e = hipGraphLaunch(ge, st);
    if (e == hipSuccess) e = hipEventRecord(t1, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    float ms = 0.f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, t0, t1);
    (void)hipEventDestroy(t0);
    (void)hipEventDestroy(t1);
    (void)hipGraphExecDestroy(ge);
    (void)hipGraphDestroy(g);
    COEUS_HIP(e);
    *ms_out = ms;
    if (launches_out) *launches_out = launches * reps;
    if (bytes_out) *bytes_out = bytes * reps;
    return COEUS_OK;
}

}  // namespace coeus
