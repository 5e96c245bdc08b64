/*
 * coeus_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE (see coeus_oracle.h).
 *
 * CPU restatement of rustllm-core/plugins/model-transformer/src/lib.rs (MT) and of
 * Transformer250MConfig in rustllm-core/src/core/model.rs (CM).  Build with
 *   gcc -O2 -ffp-contract=off -fno-fast-math -fopenmp
 * so every a*b+c stays a separate multiply and add, as in the reference.
 */
#include "coeus_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

static int g_threads = 1;
/* Threads only ever split independent output rows; results do not depend on the count. */
void orc_set_threads(int n) { g_threads = n < 1 ? 1 : n; }

/* ------------------------------------------------------------------ config */

/* CM:534-550 */
void orc_config_default(orc_config *c) {
    memset(c, 0, sizeof(*c));
    c->hidden_dim = 768;
    c->num_layers = 12;
    c->num_heads = 12;
    c->intermediate_dim = 3072;
    c->vocab_size = 50257;
    c->max_seq_len = 1024;
    c->dropout = 0.1f;
    c->attention_dropout = 0.1f;
    c->layer_norm_eps = 1e-5f;
    c->use_bias = 1;
}

/* CM:487-531 (the inherent validate, which is the one build() calls, MT:590).
 * num_heads == 0 is a division by zero in the reference (CM:498); reported as invalid here. */
int orc_config_validate(const orc_config *c, const char **key) {
    const char *k = NULL;
    if (c->hidden_dim == 0) k = "hidden_dim";
    else if (c->num_heads == 0) k = "num_heads";
    else if (c->head_dim == 0 && c->hidden_dim % c->num_heads != 0) k = "hidden_dim";
    else if (c->num_layers == 0) k = "num_layers";
    else if (c->vocab_size == 0) k = "vocab_size";
    else if (c->max_seq_len == 0) k = "max_seq_len";
    else if (c->activation > 1) k = "activation";
    else if (c->norm > 1) k = "norm";
    else if (c->norm_scope > 1) k = "norm_scope";
    else if (c->weight_dtype > 3) k = "weight_dtype";
    else if (c->kv_dtype > 2) k = "kv_dtype";
    if (key) *key = k;
    return k ? ORC_INVALID_CONFIG : ORC_OK;
}

static uint64_t head_dim_of(const orc_config *c) {
    return c->head_dim ? c->head_dim : c->hidden_dim / c->num_heads;
}

/* ------------------------------------------------------------------ parameters */

/* MT:677-740 and the per-layer walk MT:839-880, generalised: the attention inner width is
 * num_heads*head_dim (== hidden_dim in the reference) and a gated FFN carries a third matrix. */
void orc_param_layout(const orc_config *c, orc_layout *L) {
    const uint64_t H = c->hidden_dim, I = c->intermediate_dim, V = c->vocab_size;
    const uint64_t inner = c->num_heads * head_dim_of(c);
    const int gated = c->activation == 1;
    uint64_t o = 0;
    memset(L, 0, sizeof(*L));
    L->inner_dim = inner;
    L->token_embed_offset = 0;
    L->token_embed_size = V * H;
    L->first_layer_offset = V * H;

    L->ln1_scale = o; o += H;
    L->ln1_bias = o;  o += H;
    L->wq = o; o += H * inner;
    L->wk = o; o += H * inner;
    L->wv = o; o += H * inner;
    L->wo = o; o += inner * H;
    if (c->use_bias) {
        L->bq = o; o += inner;
        L->bk = o; o += inner;
        L->bv = o; o += inner;
        L->bo = o; o += H;
    }
    L->ln2_scale = o; o += H;
    L->ln2_bias = o;  o += H;
    if (gated) { L->w_gate = o; o += H * I; }
    L->w_up = o;   o += H * I;
    L->w_down = o; o += I * H;
    if (c->use_bias) {
        if (gated) { L->b_gate = o; o += I; }
        L->b_up = o;   o += I;
        L->b_down = o; o += H;
    }
    L->layer_stride = o;

    L->final_ln_offset = L->first_layer_offset + c->num_layers * L->layer_stride;
    L->output_proj_offset = L->final_ln_offset + 2 * H;
    L->output_proj_size = H * V;
    L->used_params = L->output_proj_offset + L->output_proj_size;
    /* MT:541-580 also counts max_seq_len*H "position embeddings" (MT:546) and, with bias,
     * a vocab-sized output bias (MT:575-577); neither is ever read by forward. */
    L->total_params = L->used_params + c->max_seq_len * H + (c->use_bias ? V : 0);
}

uint64_t orc_num_parameters(const orc_config *c) {
    orc_layout L;
    orc_param_layout(c, &L);
    return L.total_params;
}

/* MT:604-611: param[i] = clamp(sin((i as f32) * 0.1234567) * sqrt(2/hidden), -0.1, 0.1) */
void orc_init_default(float *params, uint64_t n, uint64_t hidden_dim) {
    const float hidden = (float)hidden_dim;
    const float scale = sqrtf(2.0f / hidden);
    for (uint64_t i = 0; i < n; i++) {
        float v = sinf((float)i * 0.1234567f) * scale;
        /* f32::clamp: NaN passes through, otherwise max(min) */
        if (v < -0.1f) v = -0.1f;
        if (v > 0.1f) v = 0.1f;
        params[i] = v;
    }
}

/* ------------------------------------------------------------------ math */

#define ORC_MIN(a, b) ((a) < (b) ? (a) : (b))

/* MT:50-74 */
void orc_matmul_ref(const float *a, const float *b, uint64_t m, uint64_t n, uint64_t k,
                    float *c) {
    const uint64_t BS = 64;
    for (uint64_t i = 0; i < m * n; i++) c[i] = 0.0f;
    for (uint64_t ii = 0; ii < m; ii += BS)
        for (uint64_t jj = 0; jj < n; jj += BS)
            for (uint64_t kk = 0; kk < k; kk += BS) {
                const uint64_t i_end = ORC_MIN(ii + BS, m);
                const uint64_t j_end = ORC_MIN(jj + BS, n);
                const uint64_t k_end = ORC_MIN(kk + BS, k);
                for (uint64_t i = ii; i < i_end; i++)
                    for (uint64_t j = jj; j < j_end; j++) {
                        float sum = c[i * n + j];
                        for (uint64_t l = kk; l < k_end; l++) sum += a[i * k + l] * b[l * n + j];
                        c[i * n + j] = sum;
                    }
            }
}

/* Each c[i,j] starts at 0 and receives a[i,l]*b[l,j] for l = 0..k-1 in ascending order,
 * every product rounded to f32 before the add: the same value sequence as MT:63-67. */
void orc_matmul(const float *a, const float *b, uint64_t m, uint64_t n, uint64_t k, float *c) {
#pragma omp parallel for schedule(static) num_threads(g_threads) if (g_threads > 1 && m > 1)
    for (int64_t i = 0; i < (int64_t)m; i++) {
        float *restrict ci = c + (uint64_t)i * n;
        for (uint64_t j = 0; j < n; j++) ci[j] = 0.0f;
        for (uint64_t l = 0; l < k; l++) {
            const float ail = a[(uint64_t)i * k + l];
            const float *restrict bl = b + l * n;
            for (uint64_t j = 0; j < n; j++) ci[j] += ail * bl[j];
        }
    }
}

/* MT:80-88.  exp is evaluated twice per element, once for the sum and once for the output. */
void orc_softmax(const float *in, uint64_t n, float *out) {
    float max_val = -INFINITY;
    for (uint64_t i = 0; i < n; i++) max_val = fmaxf(max_val, in[i]); /* f32::max */
    float exp_sum = 0.0f;
    for (uint64_t i = 0; i < n; i++) exp_sum += expf(in[i] - max_val);
    for (uint64_t i = 0; i < n; i++) out[i] = expf(in[i] - max_val) / exp_sum;
}

/* MT:94-99 */
float orc_gelu(float x) {
    const float SQRT_2_OVER_PI = 0.7978845608028654f;
    const float COEFF = 0.044715f;
    return 0.5f * x * (1.0f + tanhf(SQRT_2_OVER_PI * x * (1.0f + COEFF * x * x)));
}

/* MT:105-128.  Statistics run over the whole slice handed in. */
void orc_layer_norm(const float *in, uint64_t n, const float *scale, uint64_t n_scale,
                    const float *bias, uint64_t n_bias, float eps, float *out) {
    float mean = 0.0f, m2 = 0.0f;
    for (uint64_t i = 0; i < n; i++) {
        const float x = in[i];
        const float delta = x - mean;
        mean += delta / (float)(i + 1);
        const float delta2 = x - mean;
        m2 += delta * delta2;
    }
    const float variance = m2 / (float)n;
    const float std_dev = sqrtf(variance + eps);
    for (uint64_t i = 0; i < n; i++)
        out[i] = scale[i % n_scale] * (in[i] - mean) / std_dev + bias[i % n_bias];
}

/* Extension (no reference counterpart): y = scale * x / sqrt(mean(x^2) + eps). */
static void rms_norm(const float *in, uint64_t n, const float *scale, float eps, float *out) {
    float ss = 0.0f;
    for (uint64_t i = 0; i < n; i++) ss += in[i] * in[i];
    const float r = sqrtf(ss / (float)n + eps);
    for (uint64_t i = 0; i < n; i++) out[i] = scale[i] * in[i] / r;
}

/* ------------------------------------------------------------------ components */

/* MT:398-407 */
void orc_positional_encoding(uint64_t max_seq_len, uint64_t hidden_dim, float *t) {
    memset(t, 0, sizeof(float) * max_seq_len * hidden_dim);
    for (uint64_t pos = 0; pos < max_seq_len; pos++)
        for (uint64_t i = 0; i < hidden_dim / 2; i++) {
            const float angle =
                (float)pos / powf(10000.0f, 2.0f * (float)i / (float)hidden_dim);
            t[pos * hidden_dim + 2 * i] = sinf(angle);
            t[pos * hidden_dim + 2 * i + 1] = cosf(angle);
        }
}

/* MT:746-756 */
void orc_causal_mask(uint64_t s, float *mask) {
    memset(mask, 0, sizeof(float) * s * s);
    for (uint64_t i = 0; i < s; i++)
        for (uint64_t j = 0; j <= i; j++) mask[i * s + j] = 1.0f;
}

typedef void (*matmul_fn)(const float *, const float *, uint64_t, uint64_t, uint64_t, float *);
static matmul_fn g_matmul = orc_matmul;

static float *falloc(uint64_t n) {
    float *p = (float *)malloc(sizeof(float) * (n ? n : 1));
    if (!p) abort();
    return p;
}

/* MT:219-278: per-head copy, scores, mask, row softmax, P.V.  Generalised only in that the
 * projected width (inner = heads*head_dim) may differ from hidden_dim. */
static void attention_heads(const float *q_proj, const float *k_proj, const float *v_proj,
                            uint64_t num_heads, uint64_t head_dim, uint64_t inner,
                            const float *mask, uint64_t seq_len, float *attention_output) {
#pragma omp parallel for schedule(dynamic) num_threads(g_threads) if (g_threads > 1)
    for (int64_t head = 0; head < (int64_t)num_heads; head++) {
        const uint64_t head_start = (uint64_t)head * head_dim;
        float *q_head = falloc(seq_len * head_dim);
        float *k_head = falloc(seq_len * head_dim);
        float *v_head = falloc(seq_len * head_dim);
        float *scores = falloc(seq_len * seq_len);
        float *row = falloc(seq_len);
        for (uint64_t i = 0; i < seq_len; i++)
            for (uint64_t j = 0; j < head_dim; j++) {
                q_head[i * head_dim + j] = q_proj[i * inner + head_start + j];
                k_head[i * head_dim + j] = k_proj[i * inner + head_start + j];
                v_head[i * head_dim + j] = v_proj[i * inner + head_start + j];
            }
        const float scale = 1.0f / sqrtf((float)head_dim);
        for (uint64_t i = 0; i < seq_len; i++)
            for (uint64_t j = 0; j < seq_len; j++) {
                float score = 0.0f;
                for (uint64_t k = 0; k < head_dim; k++)
                    score += q_head[i * head_dim + k] * k_head[j * head_dim + k];
                scores[i * seq_len + j] = score * scale;
            }
        if (mask)
            for (uint64_t i = 0; i < seq_len * seq_len; i++)
                if (mask[i] == 0.0f) scores[i] = -INFINITY;
        for (uint64_t i = 0; i < seq_len; i++) {
            orc_softmax(scores + i * seq_len, seq_len, row);
            memcpy(scores + i * seq_len, row, sizeof(float) * seq_len);
        }
        for (uint64_t i = 0; i < seq_len; i++)
            for (uint64_t j = 0; j < head_dim; j++) {
                float output_val = 0.0f;
                for (uint64_t k = 0; k < seq_len; k++)
                    output_val += scores[i * seq_len + k] * v_head[k * head_dim + j];
                attention_output[i * inner + head_start + j] = output_val;
            }
        free(q_head); free(k_head); free(v_head); free(scores); free(row);
    }
}

static void add_row_bias(float *x, uint64_t rows, uint64_t width, const float *b) {
    for (uint64_t i = 0; i < rows * width; i++) x[i] = x[i] + b[i % width];
}

/* MT:167-300 */
void orc_mha_forward(uint64_t hidden_dim, uint64_t num_heads, const float *query,
                     const float *key, const float *value, const float *weights,
                     const float *bias, const float *mask, uint64_t seq_len, float *out) {
    const uint64_t H = hidden_dim, HH = H * H, head_dim = H / num_heads;
    const float *q_w = weights, *k_w = weights + HH, *v_w = weights + 2 * HH,
                *o_w = weights + 3 * HH;
    float *q_proj = falloc(seq_len * H), *k_proj = falloc(seq_len * H),
          *v_proj = falloc(seq_len * H), *attn = falloc(seq_len * H);
    g_matmul(query, q_w, seq_len, H, H, q_proj);
    g_matmul(key, k_w, seq_len, H, H, k_proj);
    g_matmul(value, v_w, seq_len, H, H, v_proj);
    if (bias) {
        add_row_bias(q_proj, seq_len, H, bias);
        add_row_bias(k_proj, seq_len, H, bias + H);
        add_row_bias(v_proj, seq_len, H, bias + 2 * H);
    }
    memset(attn, 0, sizeof(float) * seq_len * H);
    attention_heads(q_proj, k_proj, v_proj, num_heads, head_dim, H, mask, seq_len, attn);
    g_matmul(attn, o_w, seq_len, H, H, out);
    if (bias) add_row_bias(out, seq_len, H, bias + 3 * H);
    free(q_proj); free(k_proj); free(v_proj); free(attn);
}

/* MT:328-378 */
void orc_ffn_forward(uint64_t hidden_dim, uint64_t intermediate_dim, const float *input,
                     const float *weights, const float *bias, uint64_t seq_len, float *out) {
    const uint64_t H = hidden_dim, I = intermediate_dim;
    const float *up_w = weights, *down_w = weights + H * I;
    float *inter = falloc(seq_len * I);
    g_matmul(input, up_w, seq_len, I, H, inter);
    if (bias)
        for (uint64_t i = 0; i < seq_len * I; i++) inter[i] += bias[i % I];
    for (uint64_t i = 0; i < seq_len * I; i++) inter[i] = orc_gelu(inter[i]);
    g_matmul(inter, down_w, seq_len, H, I, out);
    if (bias)
        for (uint64_t i = 0; i < seq_len * H; i++) out[i] += bias[I + i % H];
    free(inter);
}

/* MT:453-499 */
void orc_block_forward(uint64_t hidden_dim, uint64_t num_heads, uint64_t intermediate_dim,
                       const float *input, const float *attn_w, const float *attn_b,
                       const float *ff_w, const float *ff_b, const float *ln1_s,
                       const float *ln1_b, const float *ln2_s, const float *ln2_b,
                       const float *mask, uint64_t seq_len, float eps, float *out) {
    const uint64_t H = hidden_dim, n = seq_len * H;
    float *normed1 = falloc(n), *attn_out = falloc(n), *normed2 = falloc(n), *ff = falloc(n);
    orc_layer_norm(input, n, ln1_s, H, ln1_b, H, eps, normed1);
    orc_mha_forward(H, num_heads, normed1, normed1, normed1, attn_w, attn_b, mask, seq_len,
                    attn_out);
    for (uint64_t i = 0; i < n; i++) out[i] = input[i] + attn_out[i];
    orc_layer_norm(out, n, ln2_s, H, ln2_b, H, eps, normed2);
    orc_ffn_forward(H, intermediate_dim, normed2, ff_w, ff_b, seq_len, ff);
    for (uint64_t i = 0; i < n; i++) out[i] += ff[i];
    free(normed1); free(attn_out); free(normed2); free(ff);
}

/* ------------------------------------------------------------------ number formats */

float orc_bf16_round(float x) {
    uint32_t u;
    memcpy(&u, &x, 4);
    if ((u & 0x7f800000u) == 0x7f800000u && (u & 0x007fffffu)) { /* NaN */
        u |= 0x00400000u;
        u &= 0xffff0000u;
    } else {
        u += 0x7fffu + ((u >> 16) & 1u);
        u &= 0xffff0000u;
    }
    memcpy(&x, &u, 4);
    return x;
}

uint16_t orc_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t absx = x & 0x7fffffffu;
    if (absx >= 0x7f800000u) /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | (absx > 0x7f800000u ? 0x0200u : 0));
    if (absx >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* rounds to >= 65520 -> inf */
    if (absx < 0x33000001u) return (uint16_t)sign;               /* below half the least subnormal */
    int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t man = (absx & 0x007fffffu) | 0x00800000u;
    uint32_t shift, half;
    if (e < -14) { /* subnormal result */
        shift = (uint32_t)(13 + (-14 - e));
        half = 0;
    } else {
        shift = 13;
        half = (uint32_t)(e + 15) << 10;
    }
    uint32_t q = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u);
    const uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) q++;
    if (e < -14) return (uint16_t)(sign | q); /* q may carry into the normal range: still right */
    return (uint16_t)(sign | (half + q - 0x400u));
}

float orc_f16_to_f32(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1fu;
    const uint32_t man = h & 0x3ffu;
    uint32_t out;
    if (exp == 0) {
        if (man == 0) out = sign;
        else {
            float v = (float)man * 5.9604644775390625e-08f; /* 2^-24 */
            memcpy(&out, &v, 4);
            out |= sign;
        }
    } else if (exp == 31) out = sign | 0x7f800000u | (man << 13);
    else out = sign | ((exp + 112u) << 23) | (man << 13);
    float f;
    memcpy(&f, &out, 4);
    return f;
}

float orc_f16_round(float x) { return orc_f16_to_f32(orc_f32_to_f16(x)); }

/* d = f16(amax/127); id = 1/f32(amax/127) as in GGML's reference quantiser: the scale is
 * taken before rounding it to f16. */
void orc_quantize_q8_0(const float *x, uint64_t n, int8_t *qs, uint16_t *ds) {
    for (uint64_t b = 0; b < n / 32; b++) {
        const float *xb = x + b * 32;
        float amax = 0.0f;
        for (int j = 0; j < 32; j++) amax = fmaxf(amax, fabsf(xb[j]));
        const float d = amax / 127.0f;
        const float id = d != 0.0f ? 1.0f / d : 0.0f;
        ds[b] = orc_f32_to_f16(d);
        for (int j = 0; j < 32; j++) qs[b * 32 + j] = (int8_t)roundf(xb[j] * id);
    }
}

void orc_dequantize_q8_0(const int8_t *qs, const uint16_t *ds, uint64_t n, float *out) {
    for (uint64_t b = 0; b < n / 32; b++) {
        const float d = orc_f16_to_f32(ds[b]);
        for (int j = 0; j < 32; j++) out[b * 32 + j] = (float)qs[b * 32 + j] * d;
    }
}

void orc_quantize_q4_0(const float *x, uint64_t n, uint8_t *qs, uint16_t *ds) {
    for (uint64_t b = 0; b < n / 32; b++) {
        const float *xb = x + b * 32;
        float amax = 0.0f, max = 0.0f;
        for (int j = 0; j < 32; j++) {
            const float v = xb[j];
            if (amax < fabsf(v)) { amax = fabsf(v); max = v; }
        }
        const float d = max / -8.0f;
        const float id = d != 0.0f ? 1.0f / d : 0.0f;
        ds[b] = orc_f32_to_f16(d);
        for (int j = 0; j < 16; j++) {
            const float x0 = xb[j] * id, x1 = xb[j + 16] * id;
            int q0 = (int)(int8_t)(x0 + 8.5f), q1 = (int)(int8_t)(x1 + 8.5f);
            if (q0 > 15) q0 = 15;
            if (q1 > 15) q1 = 15;
            qs[b * 16 + j] = (uint8_t)((unsigned)q0 | ((unsigned)q1 << 4));
        }
    }
}

void orc_dequantize_q4_0(const uint8_t *qs, const uint16_t *ds, uint64_t n, float *out) {
    for (uint64_t b = 0; b < n / 32; b++) {
        const float d = orc_f16_to_f32(ds[b]);
        for (int j = 0; j < 16; j++) {
            const int q0 = (qs[b * 16 + j] & 0x0f) - 8, q1 = (qs[b * 16 + j] >> 4) - 8;
            out[b * 32 + j] = (float)q0 * d;
            out[b * 32 + j + 16] = (float)q1 * d;
        }
    }
}

/* One [k_in, n_out] row-major matrix; blocks run along k for each output column. */
static void roundtrip_matrix(uint32_t dtype, float *w, uint64_t k_in, uint64_t n_out) {
    if (dtype == 0) return;
    if (dtype == 1) {
        for (uint64_t i = 0; i < k_in * n_out; i++) w[i] = orc_bf16_round(w[i]);
        return;
    }
    float *col = falloc(k_in), *deq = falloc(k_in);
    uint8_t *qs = (uint8_t *)malloc(k_in);
    uint16_t *ds = (uint16_t *)malloc(sizeof(uint16_t) * (k_in / 32 + 1));
    for (uint64_t j = 0; j < n_out; j++) {
        for (uint64_t l = 0; l < k_in; l++) col[l] = w[l * n_out + j];
        if (dtype == 2) {
            orc_quantize_q8_0(col, k_in, (int8_t *)qs, ds);
            orc_dequantize_q8_0((int8_t *)qs, ds, k_in, deq);
        } else {
            orc_quantize_q4_0(col, k_in, qs, ds);
            orc_dequantize_q4_0(qs, ds, k_in, deq);
        }
        for (uint64_t l = 0; l < k_in; l++) w[l * n_out + j] = deq[l];
    }
    free(col); free(deq); free(qs); free(ds);
}

void orc_apply_weight_dtype(const orc_config *c, float *p) {
    orc_layout L;
    orc_param_layout(c, &L);
    const uint64_t H = c->hidden_dim, I = c->intermediate_dim, V = c->vocab_size,
                   inner = L.inner_dim;
    const uint32_t t = c->weight_dtype;
    if (t == 0) return;
    if (t == 1)
        for (uint64_t i = 0; i < L.token_embed_size; i++) p[i] = orc_bf16_round(p[i]);
#pragma omp parallel for schedule(dynamic) num_threads(g_threads) if (g_threads > 1)
    for (int64_t l = 0; l < (int64_t)c->num_layers; l++) {
        float *base = p + L.first_layer_offset + (uint64_t)l * L.layer_stride;
        roundtrip_matrix(t, base + L.wq, H, inner);
        roundtrip_matrix(t, base + L.wk, H, inner);
        roundtrip_matrix(t, base + L.wv, H, inner);
        roundtrip_matrix(t, base + L.wo, inner, H);
        if (c->activation == 1) roundtrip_matrix(t, base + L.w_gate, H, I);
        roundtrip_matrix(t, base + L.w_up, H, I);
        roundtrip_matrix(t, base + L.w_down, I, H);
    }
    roundtrip_matrix(t, p + L.output_proj_offset, H, V);
}

/* ------------------------------------------------------------------ synthetic data */

static uint64_t splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

static uint64_t synth_hash(uint64_t seed, uint64_t counter) {
    return splitmix64(splitmix64(seed) ^ (counter * 0xD1342543DE82EF95ull + 1));
}

/* Sum of eight uniform 16-bit integers has mean 262140 and variance 8*(2^32-1)/12;
 * 1/sqrt(that) = 1.8688124e-05. */
float orc_synth_normal(uint64_t seed, uint64_t index) {
    const uint64_t a = synth_hash(seed, 2 * index), b = synth_hash(seed, 2 * index + 1);
    int32_t s = 0;
    for (int j = 0; j < 4; j++) {
        s += (int32_t)((a >> (16 * j)) & 0xffff);
        s += (int32_t)((b >> (16 * j)) & 0xffff);
    }
    return (float)(s - 262140) * 1.8688124e-05f;
}

static int is_norm_scale(const orc_config *c, const orc_layout *L, uint64_t i) {
    const uint64_t H = c->hidden_dim;
    if (i >= L->final_ln_offset) return i < L->final_ln_offset + H;
    if (i < L->first_layer_offset) return 0;
    const uint64_t r = (i - L->first_layer_offset) % L->layer_stride;
    return (r >= L->ln1_scale && r < L->ln1_scale + H) || (r >= L->ln2_scale && r < L->ln2_scale + H);
}

void orc_init_seeded(const orc_config *c, uint64_t seed, float *params, uint64_t n) {
    orc_layout L;
    orc_param_layout(c, &L);
#pragma omp parallel for schedule(static) num_threads(g_threads) if (g_threads > 1)
    for (int64_t i = 0; i < (int64_t)n; i++) {
        const float z = 0.02f * orc_synth_normal(seed, (uint64_t)i);
        params[i] = is_norm_scale(c, &L, (uint64_t)i) ? 1.0f + z : z;
    }
}

void orc_synth_ids(uint64_t seed, uint64_t vocab, uint64_t *ids, uint64_t n) {
    for (uint64_t i = 0; i < n; i++) ids[i] = synth_hash(seed, i) % vocab;
}

/* ------------------------------------------------------------------ forward */

static float round_kv(uint32_t kv_dtype, float x) {
    return kv_dtype == 1 ? orc_f16_round(x) : kv_dtype == 2 ? orc_bf16_round(x) : x;
}

static void norm_rows(const orc_config *c, const float *in, uint64_t rows, const float *scale,
                      const float *bias, float *out) {
    const uint64_t H = c->hidden_dim;
    if (c->norm_scope == 0) {
        /* the reference hands the whole [seq*hidden] buffer to layer_norm (MT:469,488,906) */
        if (c->norm == 0) orc_layer_norm(in, rows * H, scale, H, bias, H, c->layer_norm_eps, out);
        else {
            /* whole-slice RMS with tiled scale */
            float ss = 0.0f;
            for (uint64_t i = 0; i < rows * H; i++) ss += in[i] * in[i];
            const float r = sqrtf(ss / (float)(rows * H) + c->layer_norm_eps);
            for (uint64_t i = 0; i < rows * H; i++) out[i] = scale[i % H] * in[i] / r;
        }
        return;
    }
    for (uint64_t s = 0; s < rows; s++) {
        if (c->norm == 0)
            orc_layer_norm(in + s * H, H, scale, H, bias, H, c->layer_norm_eps, out + s * H);
        else rms_norm(in + s * H, H, scale, c->layer_norm_eps, out + s * H);
    }
}

static float silu(float x) { return x / (1.0f + expf(-x)); }

/* FFN on `rows` rows; the non-gated branch is MT:328-378 with split bias pointers. */
static void ffn_rows(const orc_config *c, const orc_layout *L, const float *base,
                     const float *x, uint64_t rows, float *out) {
    const uint64_t H = c->hidden_dim, I = c->intermediate_dim;
    float *inter = falloc(rows * I);
    g_matmul(x, base + L->w_up, rows, I, H, inter);
    if (c->use_bias)
        for (uint64_t i = 0; i < rows * I; i++) inter[i] += base[L->b_up + i % I];
    if (c->activation == 0) {
        for (uint64_t i = 0; i < rows * I; i++) inter[i] = orc_gelu(inter[i]);
    } else {
        float *gate = falloc(rows * I);
        g_matmul(x, base + L->w_gate, rows, I, H, gate);
        if (c->use_bias)
            for (uint64_t i = 0; i < rows * I; i++) gate[i] += base[L->b_gate + i % I];
        for (uint64_t i = 0; i < rows * I; i++) inter[i] = silu(gate[i]) * inter[i];
        free(gate);
    }
    g_matmul(inter, base + L->w_down, rows, H, I, out);
    if (c->use_bias)
        for (uint64_t i = 0; i < rows * H; i++) out[i] += base[L->b_down + i % H];
    free(inter);
}

static int embed_rows(const orc_config *c, const float *params, const float *pe,
                      const uint64_t *ids, uint64_t n, uint64_t pos0, float *h) {
    const uint64_t H = c->hidden_dim;
    for (uint64_t i = 0; i < n; i++) {
        if (ids[i] >= c->vocab_size) return ORC_INVALID_INPUT; /* MT:816-822 */
        memcpy(h + i * H, params + ids[i] * H, sizeof(float) * H);
    }
    for (uint64_t i = 0; i < n * H; i++) h[i] += pe[pos0 * H + i]; /* MT:832-835 */
    return ORC_OK;
}

/* The reference algorithm, statement for statement (extension fields all zero). */
static int forward_reference(const orc_config *c, const float *params, const uint64_t *ids,
                             uint64_t S, float *logits_last, float *logits_all) {
    const uint64_t H = c->hidden_dim, V = c->vocab_size, I = c->intermediate_dim;
    orc_layout L;
    orc_param_layout(c, &L);
    float *pe = falloc(c->max_seq_len * H);
    orc_positional_encoding(c->max_seq_len, H, pe);
    float *h = falloc(S * H), *h2 = falloc(S * H), *mask = falloc(S * S);
    int rc = embed_rows(c, params, pe, ids, S, 0, h);
    if (rc == ORC_OK) {
        for (uint64_t l = 0; l < c->num_layers; l++) {
            uint64_t off = L.first_layer_offset + l * L.layer_stride; /* MT:839-880 */
            const float *ln1_s = params + off; off += H;
            const float *ln1_b = params + off; off += H;
            const float *attn_w = params + off; off += 4 * H * H;
            const float *attn_b = NULL;
            if (c->use_bias) { attn_b = params + off; off += 4 * H; }
            const float *ln2_s = params + off; off += H;
            const float *ln2_b = params + off; off += H;
            const float *ff_w = params + off; off += 2 * H * I;
            const float *ff_b = c->use_bias ? params + off : NULL;
            orc_causal_mask(S, mask); /* MT:883 */
            orc_block_forward(H, c->num_heads, I, h, attn_w, attn_b, ff_w, ff_b, ln1_s, ln1_b,
                              ln2_s, ln2_b, mask, S, c->layer_norm_eps, h2);
            float *t = h; h = h2; h2 = t;
        }
        const float *fs = params + L.final_ln_offset, *fb = fs + H; /* MT:903-911 */
        orc_layer_norm(h, S * H, fs, H, fb, H, c->layer_norm_eps, h2);
        const float *wout = params + L.output_proj_offset;
        if (logits_last) g_matmul(h2 + (S - 1) * H, wout, 1, V, H, logits_last); /* MT:915-916 */
        if (logits_all) g_matmul(h2, wout, S, V, H, logits_all);
    }
    free(pe); free(h); free(h2); free(mask);
    return rc;
}

/* Generalised forward: same dataflow with the extension switches honoured. */
static int forward_general(const orc_config *c, const float *params, const uint64_t *ids,
                           uint64_t S, float *logits_last, float *logits_all) {
    const uint64_t H = c->hidden_dim, V = c->vocab_size;
    orc_layout L;
    orc_param_layout(c, &L);
    const uint64_t inner = L.inner_dim, hd = head_dim_of(c);
    float *pe = falloc(c->max_seq_len * H);
    orc_positional_encoding(c->max_seq_len, H, pe);
    float *h = falloc(S * H), *x = falloc(S * H), *t = falloc(S * H), *mask = falloc(S * S);
    float *q = falloc(S * inner), *k = falloc(S * inner), *v = falloc(S * inner),
          *a = falloc(S * inner);
    int rc = embed_rows(c, params, pe, ids, S, 0, h);
    if (rc == ORC_OK) {
        for (uint64_t l = 0; l < c->num_layers; l++) {
            const float *base = params + L.first_layer_offset + l * L.layer_stride;
            norm_rows(c, h, S, base + L.ln1_scale, base + L.ln1_bias, x);
            g_matmul(x, base + L.wq, S, inner, H, q);
            g_matmul(x, base + L.wk, S, inner, H, k);
            g_matmul(x, base + L.wv, S, inner, H, v);
            if (c->use_bias) {
                add_row_bias(q, S, inner, base + L.bq);
                add_row_bias(k, S, inner, base + L.bk);
                add_row_bias(v, S, inner, base + L.bv);
            }
            if (c->kv_dtype)
                for (uint64_t i = 0; i < S * inner; i++) {
                    k[i] = round_kv(c->kv_dtype, k[i]);
                    v[i] = round_kv(c->kv_dtype, v[i]);
                }
            orc_causal_mask(S, mask);
            memset(a, 0, sizeof(float) * S * inner);
            attention_heads(q, k, v, c->num_heads, hd, inner, mask, S, a);
            g_matmul(a, base + L.wo, S, H, inner, t);
            if (c->use_bias) add_row_bias(t, S, H, base + L.bo);
            for (uint64_t i = 0; i < S * H; i++) h[i] = h[i] + t[i];
            norm_rows(c, h, S, base + L.ln2_scale, base + L.ln2_bias, x);
            ffn_rows(c, &L, base, x, S, t);
            for (uint64_t i = 0; i < S * H; i++) h[i] += t[i];
        }
        const float *fs = params + L.final_ln_offset;
        norm_rows(c, h, S, fs, fs + H, x);
        const float *wout = params + L.output_proj_offset;
        if (logits_last) g_matmul(x + (S - 1) * H, wout, 1, V, H, logits_last);
        if (logits_all) g_matmul(x, wout, S, V, H, logits_all);
    }
    free(pe); free(h); free(x); free(t); free(mask); free(q); free(k); free(v); free(a);
    return rc;
}

/* flags: bit0 = use orc_matmul instead of orc_matmul_ref; bit1 = take the generalised path even
 * when every extension field is zero (used to prove both paths agree bit for bit). */
int orc_forward(const orc_config *c, const float *params, uint64_t n_params,
                const uint64_t *ids, uint64_t S, float *logits_last, float *logits_all,
                int flags) {
    orc_layout L;
    if (orc_config_validate(c, NULL) != ORC_OK) return ORC_INVALID_CONFIG;
    orc_param_layout(c, &L);
    if (S == 0 || S > c->max_seq_len) return ORC_INVALID_INPUT; /* MT:797-802 (+ empty) */
    if (n_params < L.used_params) return ORC_INVALID_INPUT;     /* MT:661-669 */
    g_matmul = (flags & 1) ? orc_matmul : orc_matmul_ref;
    const int reference_mode = !c->activation && !c->norm && !c->norm_scope && !c->kv_dtype &&
                               (c->head_dim == 0 || c->head_dim * c->num_heads == c->hidden_dim);
    int rc;
    if (reference_mode && !(flags & 2)) rc = forward_reference(c, params, ids, S, logits_last, logits_all);
    else rc = forward_general(c, params, ids, S, logits_last, logits_all);
    g_matmul = orc_matmul;
    return rc;
}

/* ------------------------------------------------------------------ KV-cache session */

struct orc_session {
    orc_config cfg;
    orc_layout L;
    const float *params;
    uint64_t max_ctx, pos;
    float *pe;
    float *kc, *vc; /* [layer][max_ctx][inner] */
    int literal;
};

orc_session *orc_session_create(const orc_config *c, const float *params, uint64_t n_params,
                                uint64_t max_ctx) {
    orc_layout L;
    if (orc_config_validate(c, NULL) != ORC_OK || c->norm_scope != 1) return NULL;
    orc_param_layout(c, &L);
    if (n_params < L.used_params || max_ctx == 0 || max_ctx > c->max_seq_len) return NULL;
    orc_session *s = (orc_session *)calloc(1, sizeof(*s));
    s->cfg = *c;
    s->L = L;
    s->params = params;
    s->max_ctx = max_ctx;
    s->pe = falloc(c->max_seq_len * c->hidden_dim);
    orc_positional_encoding(c->max_seq_len, c->hidden_dim, s->pe);
    s->kc = (float *)calloc(c->num_layers * max_ctx * L.inner_dim, sizeof(float));
    s->vc = (float *)calloc(c->num_layers * max_ctx * L.inner_dim, sizeof(float));
    if (!s->kc || !s->vc) abort();
    return s;
}

void orc_session_destroy(orc_session *s) {
    if (!s) return;
    free(s->pe); free(s->kc); free(s->vc); free(s);
}
void orc_session_reset(orc_session *s) { s->pos = 0; }
/* Timing aid: declares the first `pos` cache rows valid without computing them (they hold
 * zeros unless fed before); the arithmetic per fed token is that of a context of that length. */
int orc_session_seek(orc_session *s, uint64_t pos) {
    if (pos > s->max_ctx) return ORC_INVALID_INPUT;
    s->pos = pos;
    return ORC_OK;
}
/* 1 = run the session's matmuls through the literal loops of MT:50-74 (orc_matmul_ref). */
void orc_session_set_literal_matmul(orc_session *s, int on) { s->literal = on; }
uint64_t orc_session_position(const orc_session *s) { return s->pos; }

int orc_session_feed(orc_session *s, const uint64_t *ids, uint64_t n, float *logits_last,
                     float *logits_all) {
    const orc_config *c = &s->cfg;
    const orc_layout *L = &s->L;
    const uint64_t H = c->hidden_dim, V = c->vocab_size, inner = L->inner_dim,
                   hd = head_dim_of(c), pos0 = s->pos;
    if (n == 0 || pos0 + n > s->max_ctx) return ORC_INVALID_INPUT;
    float *h = falloc(n * H), *x = falloc(n * H), *t = falloc(n * H);
    float *q = falloc(n * inner), *k = falloc(n * inner), *v = falloc(n * inner),
          *a = falloc(n * inner);
    g_matmul = s->literal ? orc_matmul_ref : orc_matmul;
    int rc = embed_rows(c, s->params, s->pe, ids, n, pos0, h);
    if (rc == ORC_OK) {
        const float scale = 1.0f / sqrtf((float)hd);
        for (uint64_t l = 0; l < c->num_layers; l++) {
            const float *base = s->params + L->first_layer_offset + l * L->layer_stride;
            float *kc = s->kc + l * s->max_ctx * inner, *vc = s->vc + l * s->max_ctx * inner;
            norm_rows(c, h, n, base + L->ln1_scale, base + L->ln1_bias, x);
            g_matmul(x, base + L->wq, n, inner, H, q);
            g_matmul(x, base + L->wk, n, inner, H, k);
            g_matmul(x, base + L->wv, n, inner, H, v);
            if (c->use_bias) {
                add_row_bias(q, n, inner, base + L->bq);
                add_row_bias(k, n, inner, base + L->bk);
                add_row_bias(v, n, inner, base + L->bv);
            }
            for (uint64_t i = 0; i < n * inner; i++) {
                kc[pos0 * inner + i] = round_kv(c->kv_dtype, k[i]);
                vc[pos0 * inner + i] = round_kv(c->kv_dtype, v[i]);
            }
#pragma omp parallel for schedule(dynamic) num_threads(g_threads) if (g_threads > 1)
            for (int64_t hh = 0; hh < (int64_t)c->num_heads; hh++) {
                const uint64_t hs = (uint64_t)hh * hd;
                float *sc = falloc(pos0 + n), *pr = falloc(pos0 + n);
                for (uint64_t i = 0; i < n; i++) {
                    const uint64_t ctx = pos0 + i + 1; /* causal: keys 0..pos0+i */
                    for (uint64_t j = 0; j < ctx; j++) {
                        float score = 0.0f;
                        for (uint64_t d = 0; d < hd; d++)
                            score += q[i * inner + hs + d] * kc[j * inner + hs + d];
                        sc[j] = score * scale;
                    }
                    orc_softmax(sc, ctx, pr);
                    for (uint64_t d = 0; d < hd; d++) {
                        float o = 0.0f;
                        for (uint64_t j = 0; j < ctx; j++) o += pr[j] * vc[j * inner + hs + d];
                        a[i * inner + hs + d] = o;
                    }
                }
                free(sc); free(pr);
            }
            g_matmul(a, base + L->wo, n, H, inner, t);
            if (c->use_bias) add_row_bias(t, n, H, base + L->bo);
            for (uint64_t i = 0; i < n * H; i++) h[i] = h[i] + t[i];
            norm_rows(c, h, n, base + L->ln2_scale, base + L->ln2_bias, x);
            ffn_rows(c, L, base, x, n, t);
            for (uint64_t i = 0; i < n * H; i++) h[i] += t[i];
        }
        const float *fs = s->params + L->final_ln_offset;
        norm_rows(c, h, n, fs, fs + H, x);
        const float *wout = s->params + L->output_proj_offset;
        if (logits_last) g_matmul(x + (n - 1) * H, wout, 1, V, H, logits_last);
        if (logits_all) g_matmul(x, wout, n, V, H, logits_all);
        s->pos = pos0 + n;
    }
    g_matmul = orc_matmul;
    free(h); free(x); free(t); free(q); free(k); free(v); free(a);
    return rc;
}

/* ------------------------------------------------------------------ sampling (see the header) */

/* exp(x) for x <= 0 from f32 multiplies, adds and one exact power-of-two scaling: Cody-Waite
 * reduction x = n ln2 + r, |r| <= ln2/2, degree-7 Taylor polynomial in Horner form.  Relative
 * error below 2e-7; what matters is that it is reproducible bit for bit (this file and the device
 * source are compiled without floating-point contraction). */
float orc_exp_nonpositive(float x) {
    if (!(x > -87.0f)) return 0.0f;
    if (x > 0.0f) x = 0.0f;
    const float n = rintf(x * 1.44269504f);
    float r = x - n * 0.693359375f;
    r = r - n * -2.12194440e-4f;
    float p = 1.0f / 5040.0f;
    p = p * r + 1.0f / 720.0f;
    p = p * r + 1.0f / 120.0f;
    p = p * r + 1.0f / 24.0f;
    p = p * r + 1.0f / 6.0f;
    p = p * r + 0.5f;
    p = p * r + 1.0f;
    p = p * r + 1.0f;
    return ldexpf(p, (int)n);
}

uint32_t orc_sample_u24(uint64_t seed, uint64_t position, uint64_t row) {
    const uint64_t x = seed ^ ((position + 1) * 0xD1B54A32D192ED03ull) ^ ((row + 1) * 0x9E3779B97F4A7C15ull);
    return (uint32_t)(splitmix64(x) >> 40);
}

static uint64_t sample_weight(float z, float zmax, float temperature) {
    return (uint64_t)(orc_exp_nonpositive((z - zmax) / temperature) * 16777216.0f);
}

uint64_t orc_sample(const float *logits, uint64_t vocab, uint32_t top_k, float top_p, float temperature,
                    uint64_t seed, uint64_t position, uint64_t row) {
    /* NaN logits are never chosen: the greatest of the others (lowest index on ties), index 0 for
     * a row of nothing but NaN */
    uint64_t best = 0;
    int have_best = 0;
    for (uint64_t i = 0; i < vocab; i++) {
        if (logits[i] != logits[i]) continue;
        if (!have_best || logits[i] > logits[best]) { best = i; have_best = 1; }
    }
    if (!(temperature > 0.0f) || vocab == 1) return best;
    const uint64_t u24 = orc_sample_u24(seed, position, row);
    const float zmax = logits[best];
    if (top_k == 0) {
        uint64_t total = 0;
        for (uint64_t i = 0; i < vocab; i++) total += sample_weight(logits[i], zmax, temperature);
        const uint64_t target = (u24 * total) >> 24;
        uint64_t run = 0;
        for (uint64_t i = 0; i < vocab; i++) {
            run += sample_weight(logits[i], zmax, temperature);
            if (run > target) return i;
        }
        return best;
    }
    /* the top_k candidates in (value descending, index ascending) order: repeated selection of
     * the greatest element that comes after the previous one in that order */
    uint64_t k = top_k < vocab ? top_k : vocab, cand[64], w[64];
    if (k > 64) k = 64;
    float pv = 0.0f;
    uint64_t pi = 0;
    for (uint64_t j = 0; j < k; j++) {
        int have = 0;
        uint64_t bi = 0;
        for (uint64_t i = 0; i < vocab; i++) {
            const float z = logits[i];
            if (z != z) continue;
            if (j > 0 && !(z < pv || (z == pv && i > pi))) continue;
            if (!have || z > logits[bi]) { bi = i; have = 1; }
        }
        if (!have) { k = j; break; }  /* NaNs or fewer elements than asked for */
        cand[j] = bi;
        pv = logits[bi];
        pi = bi;
    }
    if (k == 0) return best;  /* no candidate at all (a row of NaN) */
    uint64_t total = 0;
    for (uint64_t j = 0; j < k; j++) { w[j] = sample_weight(logits[cand[j]], zmax, temperature); total += w[j]; }
    uint64_t m = k;
    if (top_p > 0.0f && top_p < 1.0f) {
        const uint64_t thr = ((uint64_t)(top_p * 16777216.0f) * total) >> 24;
        uint64_t run = 0;
        for (m = 0; m < k;) {
            run += w[m++];
            if (run >= thr) break;
        }
        total = run;
    }
    const uint64_t target = (u24 * total) >> 24;
    uint64_t run = 0;
    for (uint64_t j = 0; j < m; j++) {
        run += w[j];
        if (run > target) return cand[j];
    }
    return cand[0];
}
