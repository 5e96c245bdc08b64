/*
 * coeus_oracle.h -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C, single-threaded CPU restatement of the transformer forward pass of
 * rustllm-core's model-transformer plugin
 * (reference: rustllm-core/plugins/model-transformer/src/lib.rs, cited below as MT:line,
 *  and rustllm-core/src/core/model.rs, cited as CM:line).
 *
 * Only the test-suite, the smoke check and the bench's cpu_baseline leg may link or load
 * this library.  The product library (libcoeus_mi355x.so) never calls it.
 *
 * Arithmetic contract: IEEE f32, strict left-to-right evaluation, no FMA contraction
 * (compile with -ffp-contract=off, never -ffast-math), libm for sin/cos/pow/exp/tanh/sqrt.
 *
 * Parity status of each group (what pins it is listed in tests/test_oracle_*.py):
 *   pinned by reference tests / closed forms / brute force:
 *     config defaults+validate (CM:776-807), parameter count and layout (MT:541-580,677-740),
 *     default init (MT:604-611), matmul (MT:50-74), softmax (MT:80-88), gelu (MT:94-99),
 *     layer_norm (MT:105-128), positional encoding (MT:398-407), multi-head attention
 *     (MT:167-300), feed-forward (MT:328-378), block (MT:453-499), forward (MT:791-919).
 *   parity unpinned (no counterpart exists in the reference; pinned only by this build's own
 *   stated conventions and by invariants):
 *     per-token norm scope, RMSNorm, SiLU-gated FFN, decoupled head_dim, bf16 rounding,
 *     Q8_0 / Q4_0 block quantisation, KV-cache incremental decode, batching, the seeded
 *     weight generator.
 */
#ifndef COEUS_ORACLE_H
#define COEUS_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Same field meaning as Transformer250MConfig (CM:389-423) followed by extension fields.
 * All-zero extension fields reproduce the reference exactly. */
typedef struct orc_config {
    uint64_t hidden_dim, num_layers, num_heads, intermediate_dim, vocab_size, max_seq_len;
    float dropout, attention_dropout, layer_norm_eps;
    uint8_t use_bias;
    /* extensions */
    uint32_t activation;   /* 0 = GELU (tanh form, MT:94-99), 1 = SiLU-gated */
    uint32_t norm;         /* 0 = LayerNorm, 1 = RMSNorm */
    uint32_t norm_scope;   /* 0 = whole [seq*hidden] slice (reference, MT:105-128), 1 = per token */
    uint32_t weight_dtype; /* 0 = f32, 1 = bf16, 2 = Q8_0, 3 = Q4_0 (applied to linear weights) */
    uint32_t kv_dtype;     /* 0 = f32, 1 = f16, 2 = bf16 (rounding applied to cached K/V) */
    uint64_t head_dim;     /* 0 => hidden_dim / num_heads (MT:153) */
    uint64_t max_batch;    /* unused by the oracle */
} orc_config;

enum { ORC_OK = 0, ORC_INVALID_INPUT = 1, ORC_INVALID_CONFIG = 2 };

/* Worker threads for the row-parallel loops (default 1).  Threads only split independent
 * output rows / heads / layers, so results are bit-identical for any count. */
void orc_set_threads(int n);

/* ---- config (CM:534-550, CM:487-531) ---- */
void orc_config_default(orc_config *cfg);
/* Returns ORC_OK or ORC_INVALID_CONFIG; *key receives the offending field name. */
int orc_config_validate(const orc_config *cfg, const char **key);

/* ---- parameters (MT:541-580, MT:677-740, MT:604-611) ---- */
typedef struct orc_layout {
    uint64_t token_embed_offset, token_embed_size;
    uint64_t first_layer_offset, layer_stride;
    /* offsets relative to a layer's base */
    uint64_t ln1_scale, ln1_bias, wq, wk, wv, wo, bq, bk, bv, bo;
    uint64_t ln2_scale, ln2_bias, w_gate, w_up, w_down, b_gate, b_up, b_down;
    uint64_t final_ln_offset, output_proj_offset, output_proj_size;
    uint64_t used_params;  /* output_proj_offset + output_proj_size */
    uint64_t total_params; /* what build() allocates (includes the never-read tail) */
    uint64_t inner_dim;    /* num_heads * head_dim */
} orc_layout;

uint64_t orc_num_parameters(const orc_config *cfg);
void orc_param_layout(const orc_config *cfg, orc_layout *out);
void orc_init_default(float *params, uint64_t n, uint64_t hidden_dim);

/* ---- math (MT:44-129) ---- */
/* Literal restatement of the 64^3-blocked loops of MT:50-74. */
void orc_matmul_ref(const float *a, const float *b, uint64_t m, uint64_t n, uint64_t k, float *c);
/* Same per-element arithmetic (ascending-k, separate multiply and add) in i-k-j loop order so
 * the compiler can vectorise over j; bit-identical to orc_matmul_ref. */
void orc_matmul(const float *a, const float *b, uint64_t m, uint64_t n, uint64_t k, float *c);
void orc_softmax(const float *in, uint64_t n, float *out);
float orc_gelu(float x);
void orc_layer_norm(const float *in, uint64_t n, const float *scale, uint64_t n_scale,
                    const float *bias, uint64_t n_bias, float eps, float *out);

/* ---- components ---- */
/* MT:398-407 */
void orc_positional_encoding(uint64_t max_seq_len, uint64_t hidden_dim, float *table);
/* MT:746-756 */
void orc_causal_mask(uint64_t seq_len, float *mask);
/* MT:167-300.  weights = Wq|Wk|Wv|Wo consecutive, bias (nullable) = bq|bk|bv|bo, mask nullable. */
void orc_mha_forward(uint64_t hidden_dim, uint64_t num_heads, const float *query,
                     const float *key, const float *value, const float *weights,
                     const float *bias, const float *mask, uint64_t seq_len, float *out);
/* MT:328-378 */
void orc_ffn_forward(uint64_t hidden_dim, uint64_t intermediate_dim, const float *input,
                     const float *weights, const float *bias, uint64_t seq_len, float *out);
/* MT:453-499 */
void orc_block_forward(uint64_t hidden_dim, uint64_t num_heads, uint64_t intermediate_dim,
                       const float *input, const float *attn_w, const float *attn_b,
                       const float *ff_w, const float *ff_b, const float *ln1_s,
                       const float *ln1_b, const float *ln2_s, const float *ln2_b,
                       const float *mask, uint64_t seq_len, float eps, float *out);

/* ---- forward (MT:791-919) ----
 * logits_last [vocab] receives the last token's logits (what the reference returns);
 * logits_all (nullable) [seq, vocab] receives every row's logits.
 * With all extension fields zero this is the reference algorithm, statement for statement.
 * flags bit0 selects orc_matmul (1) or orc_matmul_ref (0); bit1 forces the generalised code
 * path even when every extension field is zero (to prove both paths agree bit for bit).
 * Empty input and out-of-range ids return ORC_INVALID_INPUT (the reference panics on empty
 * input, MT:915). */
int orc_forward(const orc_config *cfg, const float *params, uint64_t n_params,
                const uint64_t *ids, uint64_t seq_len, float *logits_last, float *logits_all,
                int flags);

/* ---- extensions: number formats (no counterpart in the reference) ---- */
float orc_bf16_round(float x);            /* round-to-nearest-even to bf16, back to f32 */
uint16_t orc_f32_to_f16(float x);         /* IEEE binary16, round-to-nearest-even */
float orc_f16_to_f32(uint16_t h);
float orc_f16_round(float x);
/* Q8_0: blocks of 32 along the given contiguous run; d = f16(amax/127); q = round(x/d).
 * n must be a multiple of 32.  qs[n] int8, ds[n/32] f16 bits. */
void orc_quantize_q8_0(const float *x, uint64_t n, int8_t *qs, uint16_t *ds);
void orc_dequantize_q8_0(const int8_t *qs, const uint16_t *ds, uint64_t n, float *out);
/* Q4_0: d = f16(max/-8) where max is the signed value of largest magnitude;
 * q = min(15, (int)(x/d + 8.5)); byte j of a block holds element j (low nibble) and
 * element j+16 (high nibble).  qs[n/2] bytes, ds[n/32] f16 bits. */
void orc_quantize_q4_0(const float *x, uint64_t n, uint8_t *qs, uint16_t *ds);
void orc_dequantize_q4_0(const uint8_t *qs, const uint16_t *ds, uint64_t n, float *out);
/* Replace every linear weight matrix of a flat parameter buffer (Wq,Wk,Wv,Wo,W_gate,W_up,
 * W_down, output projection) by its round trip through cfg->weight_dtype.  Quantisation
 * blocks run along the input (reduction) dimension of each output column.  The token
 * embedding is rounded to bf16 when weight_dtype is bf16 and left f32 otherwise. */
void orc_apply_weight_dtype(const orc_config *cfg, float *params);

/* ---- extensions: seeded synthetic weights ----
 * z(seed, i) = (sum of eight 16-bit lanes of splitmix64(seed, 2i) and splitmix64(seed, 2i+1)
 *               - 262140) * 1.8688124e-05f : an Irwin-Hall(8) approximation of N(0,1)
 * that is exactly reproducible in integer + one f32 multiply on any device. */
float orc_synth_normal(uint64_t seed, uint64_t index);
/* param[i] = mean(i) + 0.02 * z(seed, i); mean is 1 for norm scales, 0 elsewhere. */
void orc_init_seeded(const orc_config *cfg, uint64_t seed, float *params, uint64_t n);
/* ids[i] = splitmix64(seed, i) % vocab */
void orc_synth_ids(uint64_t seed, uint64_t vocab, uint64_t *ids, uint64_t n);

/* ---- extensions: KV-cache session (per-token norm scope only) ---- */
typedef struct orc_session orc_session;
orc_session *orc_session_create(const orc_config *cfg, const float *params, uint64_t n_params,
                                uint64_t max_ctx);
void orc_session_destroy(orc_session *s);
void orc_session_reset(orc_session *s);
uint64_t orc_session_position(const orc_session *s);
/* Timing aids for the CPU baseline: position the session at a context length without computing
 * the prefix (cache rows hold zeros), and route the matmuls through the literal MT:50-74 loops. */
int orc_session_seek(orc_session *s, uint64_t pos);
void orc_session_set_literal_matmul(orc_session *s, int on);
/* Feeds n ids at positions pos..pos+n-1, appends their K/V to the cache and writes the
 * logits of the last fed token to logits_last [vocab] (logits_all nullable, [n, vocab]). */
int orc_session_feed(orc_session *s, const uint64_t *ids, uint64_t n, float *logits_last,
                     float *logits_all);

/* ------------------------------------------------------------------ sampling
 * The reference defines only the configuration of generation (BasicGenerationConfig: temperature,
 * top_k, top_p; src/core/model.rs:718-753) and the GenerativeModel trait (model.rs:138-144); it has
 * no sampler.  This is the specification the device sampler is checked against:
 *   temperature <= 0                  -> argmax, lowest index on ties
 *   candidates                        -> the top_k largest logits (descending, ties by ascending
 *                                        index), or the whole vocabulary in index order (top_k = 0)
 *   weight w_j                        -> floor(exp((z_j - z_max) / temperature) * 2^24) with the
 *                                        exponential of orc_exp_nonpositive (f32 basic operations
 *                                        only, so every IEEE machine gets the same bits)
 *   top_p in (0, 1), top_k > 0 only   -> keep the shortest prefix of the candidates whose weight
 *                                        reaches floor(top_p * 2^24) * total >> 24 (at least one)
 *   draw                              -> u24 = top 24 bits of a counter hash of (seed, position,
 *                                        row); the first candidate whose running weight sum
 *                                        exceeds (u24 * total) >> 24
 * Everything after the weights is integer arithmetic, so summation order does not matter.  */
float orc_exp_nonpositive(float x);
uint32_t orc_sample_u24(uint64_t seed, uint64_t position, uint64_t row);
uint64_t orc_sample(const float *logits, uint64_t vocab, uint32_t top_k, float top_p, float temperature,
                    uint64_t seed, uint64_t position, uint64_t row);

#ifdef __cplusplus
}
#endif
#endif
