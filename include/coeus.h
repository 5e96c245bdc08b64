/*
 * coeus.h -- C ABI of libcoeus_mi355x.so: the transformer forward pass of rustllm-core's
 * model-transformer plugin, executed by hand-written HIP kernels on one MI355X (gfx950).
 *
 * This is the surface a Rust FFI shim (or any other host language) binds in order to replace,
 * call for call, the CPU path behind
 *     TransformerModelPlugin -> create_builder() -> build(config) -> model.forward(token_ids)
 * in rustllm-core/plugins/model-transformer/src/lib.rs (cited below as MT:line; the config
 * type lives in rustllm-core/src/core/model.rs, cited as CM:line).
 *
 * Conventions
 *   - plain pointers and sizes only; `usize` maps to uint64_t; the caller owns every in/out
 *     buffer, the library owns coeus_model / coeus_session / coeus_weight handles;
 *   - every function returning int returns a coeus_status; on failure coeus_last_error()
 *     holds a message (thread-local, valid until the next failing call on that thread);
 *   - COEUS_INVALID_INPUT maps to Error::Processing(InvalidInput{..}) and COEUS_INVALID_CONFIG
 *     to Error::Config(ConfigError::Invalid{..}) of rustllm-core/src/foundation/error.rs:17-44;
 *     the messages are the reference's own format strings;
 *   - no exception or abort crosses this boundary; a handle may be used from several threads,
 *     calls on one model or session are serialised internally (Model: Send + Sync, CM:77).
 */
#ifndef COEUS_H
#define COEUS_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum coeus_status {
    COEUS_OK = 0,
    COEUS_INVALID_INPUT = 1,
    COEUS_INVALID_CONFIG = 2,
    COEUS_DEVICE_ERROR = 3,
    COEUS_OUT_OF_MEMORY = 4
} coeus_status;

enum { COEUS_ACT_GELU_TANH = 0, COEUS_ACT_SILU_GATED = 1 };
enum { COEUS_NORM_LAYERNORM = 0, COEUS_NORM_RMSNORM = 1 };
enum { COEUS_SCOPE_SEQUENCE = 0, COEUS_SCOPE_TOKEN = 1 };
enum { COEUS_W_F32 = 0, COEUS_W_BF16 = 1, COEUS_W_Q8_0 = 2, COEUS_W_Q4_0 = 3 };
enum { COEUS_KV_F32 = 0, COEUS_KV_F16 = 1, COEUS_KV_BF16 = 2 };

/* Transformer250MConfig (CM:389-423), field for field (the `activation` string of the
 * reference is never consulted, MT:356-358, and is replaced by the enum below), followed by
 * extension fields.  All-zero extension fields select exactly the reference's behaviour:
 * tanh-GELU FFN, LayerNorm whose statistics span the whole [seq*hidden] slice (MT:105-128 as
 * called from MT:469,488,906), f32 weights, head_dim = hidden_dim / num_heads (MT:153). */
typedef struct coeus_config {
    uint64_t hidden_dim, num_layers, num_heads, intermediate_dim, vocab_size, max_seq_len;
    float dropout, attention_dropout, layer_norm_eps;
    uint8_t use_bias;
    uint32_t activation;   /* COEUS_ACT_*  */
    uint32_t norm;         /* COEUS_NORM_* */
    uint32_t norm_scope;   /* COEUS_SCOPE_*; sessions (KV cache) require COEUS_SCOPE_TOKEN */
    uint32_t weight_dtype; /* COEUS_W_*: storage of the linear weights on the device */
    uint32_t kv_dtype;     /* COEUS_KV_*: storage of cached keys/values */
    uint64_t head_dim;     /* 0 => hidden_dim / num_heads */
    uint64_t max_batch;    /* 0 => 1; upper bound for coeus_session_create's batch */
} coeus_config;

/* BasicGenerationConfig (CM:718-753) minus max_length, plus the seed of the draw.  temperature
 * <= 0 selects the greatest logit; top_k = 0 samples the whole vocabulary, else 1..64; top_p
 * outside (0, 1) is off, inside it needs top_k. */
typedef struct coeus_sampling {
    float temperature;
    uint32_t top_k;
    float top_p;
    uint64_t seed;
} coeus_sampling;

typedef struct coeus_model coeus_model;
typedef struct coeus_session coeus_session;

/* Thread-local message of the last failing call on this thread ("" if none). */
const char *coeus_last_error(void);
/* 1 when a rocprofiler tool library (rocprofv3's librocprofiler-sdk-tool.so, a roctracer or
 * rocprofiler v1/v2 library) is named by ROCP_TOOL_LIBRARIES / LD_PRELOAD / HSA_TOOLS_LIB or mapped
 * into this process; looked up once.  No counterpart in the reference. */
int coeus_profiler_attached(void);
/* Name of the device the library runs on; COEUS_DEVICE_ERROR if no gfx950 GPU is visible. */
int coeus_device_info(char *name_out, uint64_t name_cap, uint64_t *hbm_bytes, uint32_t *compute_units);

/* ---- device memory, streams, events ------------------------------------------------------
 * Thin wrappers over the HIP runtime this library is linked against, so a host (a test, a
 * bench, an FFI shim) can own device buffers and time kernels without loading a second HIP
 * runtime into the process.  No reference counterpart (the reference is CPU-only). */
int coeus_device_malloc(uint64_t bytes, void **out);
int coeus_device_free(void *ptr);
int coeus_memcpy_h2d(void *dst_dev, const void *src_host, uint64_t bytes);
int coeus_memcpy_d2h(void *dst_host, const void *src_dev, uint64_t bytes);
int coeus_device_memset(void *dst_dev, int value, uint64_t bytes);
/* Device-to-device copy by a plain kernel (device_copy_kernel: every byte read once and written
 * once, 16 bytes per lane); bytes must be a multiple of 16.  Also the reference point for the
 * memory-traffic counters: a launch of known size to scale FETCH_SIZE / WRITE_SIZE against. */
int coeus_device_copy(void *dst_dev, const void *src_dev, uint64_t bytes, void *stream);
int coeus_device_synchronize(void);
int coeus_stream_create(void **stream_out);  /* default priority, non-blocking */
int coeus_stream_synchronize(void *stream);
int coeus_stream_destroy(void *stream);
int coeus_event_create(void **event_out);
int coeus_event_record(void *event, void *stream);
int coeus_event_synchronize(void *event);
int coeus_event_elapsed_ms(void *start, void *stop, float *ms_out);
int coeus_event_destroy(void *event);

/* ---- configuration -------------------------------------------------------------------- */
/* Default for Transformer250MConfig (CM:534-550): 768/12/12/3072, vocab 50257, 1024
 * positions, dropout 0.1, eps 1e-5, bias on; extension fields zero. */
void coeus_config_default(coeus_config *cfg);
/* Transformer250MConfig::validate (CM:487-531), same order of checks.  num_heads == 0, a
 * division by zero in the reference (CM:498), is reported as invalid. */
int coeus_config_validate(const coeus_config *cfg);
/* TransformerModelBuilder::calculate_num_parameters (MT:541-580): the length of the flat
 * parameter buffer build() allocates, including the tail forward never reads. */
uint64_t coeus_config_num_parameters(const coeus_config *cfg);
/* Number of leading parameters forward actually reads (offset of the output projection plus
 * its size, MT:677-740). */
uint64_t coeus_config_used_parameters(const coeus_config *cfg);
/* ---- .rustllm files -------------------------------------------------------------------------
 * ModelSerializable for TransformerModel (MT:930-1121) over core/serialization.rs: ModelHeader
 * (:33-73, 136 bytes), ParameterSerializer (:104-190, little-endian f32), ModelMetadata
 * (:198-330) and calculate_checksum (:375-385).  The parameter buffer is the flat f32 vector that
 * coeus_model_create takes.  The writer emits the reference's five metadata keys first
 * (MT:966-971), then the other config fields under their names; the reader takes every key it
 * finds and defaults for the rest, as read_from does (MT:1062-1098).  Errors use the reference's
 * messages: "Invalid magic bytes", "Unsupported format version: N", "Checksum mismatch". */
uint64_t coeus_rustllm_checksum(const float *params, uint64_t n_params);
int coeus_rustllm_write(const char *path, const coeus_config *cfg, const float *params, uint64_t n_params);
int coeus_rustllm_read_header(const char *path, coeus_config *cfg_out, uint64_t *n_params_out);
int coeus_rustllm_read_parameters(const char *path, float *params_out, uint64_t n_params);

/* ---- byte-pair-encoding tokenizer ---------------------------------------------------------------
 * BpeTokenizer of rustllm-core/plugins/tokenizer-bpe/src/lib.rs (TB:line): the step before the
 * ids that coeus_model_forward takes.  Host code; text is UTF-8 given as pointer + length (not
 * NUL-terminated).  Text that is not valid UTF-8 returns COEUS_INVALID_INPUT (a Rust &str cannot
 * hold it).  Ids are the reference's TokenId (u32) widened to the uint64_t that forward takes.
 * Output buffers follow one protocol: the needed size is always stored through the length
 * pointer; a NULL buffer only sizes; a buffer that is too small returns COEUS_INVALID_INPUT.
 * A handle may be read (tokenize, queries) from several threads at once; train / add / remove
 * need exclusive access, as &mut self does in the reference. */
typedef struct coeus_bpe coeus_bpe;
/* BpeTokenizer::new (TB:117-143): 256 byte-level tokens (bytes >= 0x80 spelled "<0xNN>") with
 * ids 0..255, then <PAD>, <UNK>, <BOS>, <EOS> registered over ids 0..3. */
int coeus_bpe_create(coeus_bpe **out);
void coeus_bpe_destroy(coeus_bpe *t);
/* BpeTokenizer::train (TB:167-240): learns up to num_merges merge rules from the corpus (words =
 * runs of non-white-space characters; stops early when no pair is left).  Where several pairs
 * share the highest frequency the reference's pick depends on its hash map's random seed; this
 * library takes the smallest (first, second) in byte order. */
int coeus_bpe_train(coeus_bpe *t, const char *const *texts, const uint64_t *lens, uint64_t n_texts,
                    uint64_t num_merges);
/* Tokenizer::tokenize (TB:285-317): per word, bytes -> byte tokens -> every merge rule in the
 * order learned (TB:243-271) -> ids (a token missing from the vocabulary -> 1 = <UNK>), with a
 * " " token (id 32) between words.  ids [ids_cap] and n_tokens receive the ids; pieces
 * [pieces_cap], offsets [n_tokens + 1] and pieces_len the token strings back to back (the
 * StringToken values); any of ids / pieces / offsets may be NULL. */
int coeus_bpe_tokenize(const coeus_bpe *t, const char *text, uint64_t len, uint64_t *ids,
                       uint64_t ids_cap, uint64_t *n_tokens, char *pieces, uint64_t pieces_cap,
                       uint64_t *offsets, uint64_t *pieces_len);
/* Tokenizer::decode (TB:319-343) on token strings: concatenation, except that a string of the
 * form "<0x..>" becomes the single byte named by its characters 3..5 (U+FFFD if >= 0x80).  The
 * reference panics on a token such as "<0x>" (TB:329); it is copied unchanged here. */
int coeus_bpe_decode(const char *pieces, const uint64_t *offsets, uint64_t n_tokens, char *out,
                     uint64_t cap, uint64_t *len);
/* Tokenizer::vocab_size (TB:345-347) and the number of merge rules learned so far. */
uint64_t coeus_bpe_vocab_size(const coeus_bpe *t);
uint64_t coeus_bpe_num_merges(const coeus_bpe *t);
/* Merge rule `index` (the reference keeps them in a private Vec<TokenPair>, TB:107). */
int coeus_bpe_merge_rule(const coeus_bpe *t, uint64_t index, char *first, uint64_t first_cap,
                         uint64_t *first_len, char *second, uint64_t second_cap, uint64_t *second_len);
/* VocabularyTokenizer (TB:355-386): add_token returns the existing id or the next free one;
 * remove_token fails with "Token not found: .."; id_from_token / token_from_id report a missing
 * entry through *found = 0 (Option::None). */
int coeus_bpe_add_token(coeus_bpe *t, const char *token, uint64_t len, uint64_t *id_out);
int coeus_bpe_remove_token(coeus_bpe *t, const char *token, uint64_t len);
int coeus_bpe_id_from_token(const coeus_bpe *t, const char *token, uint64_t len, uint64_t *id_out,
                            int *found);
int coeus_bpe_token_from_id(const coeus_bpe *t, uint64_t id, char *out, uint64_t cap, uint64_t *len,
                            int *found);

/* The initialisation loop of build() (MT:604-611):
 * params[i] = clamp(sin((i as f32) * 0.1234567) * sqrt(2 / hidden_dim), -0.1, 0.1). */
int coeus_init_default_parameters(float *params, uint64_t n, uint64_t hidden_dim);

/* ---- model ---------------------------------------------------------------------------- */
/* Replaces TransformerModelBuilder::build (MT:587-638) for a caller that holds the flat f32
 * parameter buffer in the reference's layout (MT:677-740): validates, converts the linear
 * weights to cfg->weight_dtype, uploads everything once.  n_params must be at least
 * coeus_config_used_parameters(cfg).  The buffer is not referenced after the call returns. */
int coeus_model_create(const coeus_config *cfg, const float *params, uint64_t n_params,
                       coeus_model **out);
/* Same model shape with synthetic weights generated on the device from a counter-based
 * generator: param[i] = mean(i) + 0.02 * z(seed, i), z an Irwin-Hall(8) normal approximation,
 * mean 1 for norm scales and 0 elsewhere.  No reference counterpart (the reference has one
 * fixed init, MT:604-611); exists so multi-GB configurations need no host-side buffer. */
int coeus_model_create_seeded(const coeus_config *cfg, uint64_t seed, coeus_model **out);
/* ForwardModel::forward (MT:791-919): token ids in, the LAST token's logits out
 * (logits_out[vocab_size]).  Errors as the reference: seq_len > max_seq_len ->
 * "Sequence length {} out of range [1, {}]" (MT:797-802); id >= vocab ->
 * "Token ID {} out of range [0, {}]" (MT:816-822).  seq_len == 0, a panic in the reference
 * (MT:915), returns COEUS_INVALID_INPUT. */
int coeus_model_forward(coeus_model *m, const uint64_t *ids, uint64_t seq_len,
                        float *logits_out);
/* Same computation, logits of every row: logits_out[seq_len * vocab_size].  The reference
 * computes only the last row (MT:915-916); rows use the same final normalisation output. */
int coeus_model_forward_all(coeus_model *m, const uint64_t *ids, uint64_t seq_len,
                            float *logits_out);
/* Model::num_parameters (MT:921-923) / Model::config (MT:778-780) / Model::name (MT:782-784). */
uint64_t coeus_model_num_parameters(const coeus_model *m);
const coeus_config *coeus_model_config(const coeus_model *m);
const char *coeus_model_name(const coeus_model *m);
/* Bytes of device memory held by the model's weights. */
uint64_t coeus_model_weight_bytes(const coeus_model *m);
/* The same plus the resident f16 copies of quantised layer matrices that the prompt pass multiplies
 * with (made at build time and on first use while a 64 GiB budget lasts; 0 extra for f32 / bf16). */
uint64_t coeus_model_resident_bytes(const coeus_model *m);
void coeus_model_destroy(coeus_model *m);

/* ---- KV-cache sessions (no counterpart in the reference, which recomputes the whole
 *      sequence on every call; needs norm_scope == COEUS_SCOPE_TOKEN) ---------------------- */
int coeus_session_create(coeus_model *m, uint64_t batch, uint64_t max_ctx, coeus_session **out);
/* Feeds ids[batch][n] (row-major) at positions pos..pos+n-1 of every sequence, appends their
 * keys/values to the cache, writes the logits of the last fed token: logits_out[batch][vocab]
 * (nullable). */
int coeus_session_prefill(coeus_session *s, const uint64_t *ids, uint64_t n, float *logits_out);
/* One token per sequence: ids[batch] -> logits_out[batch][vocab]. */
int coeus_session_decode(coeus_session *s, const uint64_t *ids, float *logits_out);
/* n_steps greedy steps entirely on the device: step 0 consumes first_ids[batch], every later
 * step consumes the argmax of the previous step's logits (lowest index wins ties).
 * out_ids[batch][n_steps] receives the argmax chosen after each step. */
int coeus_session_decode_greedy(coeus_session *s, const uint64_t *first_ids, uint64_t n_steps,
                                uint64_t *out_ids);
/* The same loop with the token of every step drawn by the sampler (coeus_op_sample's rules; the
 * draw for a token is keyed by cfg->seed, the position the token takes and the sequence index):
 * GenerativeModel::generate (CM:138-144) for BasicGenerationConfig (CM:718-753).  cfg NULL or
 * temperature <= 0 is coeus_session_decode_greedy. */
int coeus_session_generate(coeus_session *s, const uint64_t *first_ids, uint64_t n_steps,
                           const coeus_sampling *cfg, uint64_t *out_ids);
/* Greedy decoding replays one captured HIP graph per step (default); 0 launches the kernels
 * one by one instead.  No counterpart in the reference.  A session created while a rocprofiler
 * tool library is loaded in the process (coeus_profiler_attached), or with COEUS_NO_GRAPH=1 in
 * the environment, starts with plain launches, and enabling graphs there is refused with
 * COEUS_INVALID_INPUT: replaying a captured decode step under rocprofv3 has ended the process
 * with a segmentation fault.  The two measurement hooks below follow the session's setting. */
int coeus_session_set_graph(coeus_session *s, int enabled);
int coeus_session_graph_enabled(const coeus_session *s);
/* Measurement hook: replays only the decode matmuls of one step (4 per layer + the logits
 * projection; real weights, shapes and epilogues) `reps` times from a captured graph and times
 * them with events on the model's stream.  *launches_out = matmul launches timed,
 * *bytes_out = algorithmic bytes they moved (stored weights + activations in and out). */
int coeus_session_time_decode_matmuls(coeus_session *s, uint64_t reps, float *ms_out,
                                      uint64_t *launches_out, uint64_t *bytes_out);
/* The same for the attention launches of one step (one per layer) over the positions cached so
 * far: *bytes_out = keys and values of every cached position of every (sequence, head) plus the
 * query and output rows.  The kernel that dominates a step at batch 16. */
int coeus_session_time_decode_attention(coeus_session *s, uint64_t reps, float *ms_out,
                                        uint64_t *launches_out, uint64_t *bytes_out);
uint64_t coeus_session_position(const coeus_session *s);
int coeus_session_reset(coeus_session *s);
void coeus_session_destroy(coeus_session *s);

/* ---- single operators on device memory ---------------------------------------------------
 * The kernels the model is built from, callable on caller-owned device buffers so each one
 * can be checked and timed in isolation.  `stream` is a hipStream_t (NULL = default stream);
 * calls only enqueue work.  Activations are f32 row-major unless stated.  Unlike models and
 * sessions, operator calls are not serialised by the library: calls that use one coeus_weight (its
 * activation staging buffer) from several threads or streams at once must be ordered by the caller. */
typedef struct coeus_weight coeus_weight;

/* A linear weight resident on the device in `dtype`.  host_w is the reference's [k_in, n_out]
 * row-major f32 matrix (b[l*n + j], MT:65); quantisation blocks of 32 run along k_in for each
 * output column (GGML block_q8_0 / block_q4_0 value convention). */
int coeus_weight_create(uint32_t dtype, const float *host_w, uint64_t k_in, uint64_t n_out,
                        coeus_weight **out);
/* Synthetic weight: element (l, j) = 0.02 * z(seed, base_index + l*n_out + j). */
int coeus_weight_create_seeded(uint32_t dtype, uint64_t seed, uint64_t base_index,
                               uint64_t k_in, uint64_t n_out, coeus_weight **out);
/* Decodes the device representation back to a host [k_in, n_out] f32 matrix. */
int coeus_weight_dequantize(const coeus_weight *w, float *host_out);
uint64_t coeus_weight_bytes(const coeus_weight *w);
void coeus_weight_destroy(coeus_weight *w);

enum { COEUS_EPI_NONE = 0, COEUS_EPI_GELU = 1, COEUS_EPI_SILU_GATE = 2 };

/* y[b, :] = epilogue(x[b, :] . W + bias) (+ residual[b, :]) for b < batch <= 16: the decode
 * matmul (MT:50-74 with m = batch).  x_dev [batch, k_in] f32, y_dev [batch, n_out] f32.
 * bias_dev / residual_dev nullable.  COEUS_EPI_SILU_GATE expects a weight created with
 * 2*n rows interleaved (gate_j, up_j) and writes n = n_out/2 values silu(gate_j)*up_j. */
int coeus_op_gemv(const coeus_weight *w, const float *x_dev, uint64_t batch, const float *bias_dev,
                  const float *residual_dev, uint32_t epilogue, float *y_dev, void *stream);
/* y[b, :] = epilogue(norm(h[b, :]) . W + bias) (+ residual[b, :]): the decode matmul with the
 * normalisation of its input rows (math::layer_norm per row, MT:105-128, or a root-mean-square
 * norm; scale_dev / bias_norm_dev [k_in]) folded into the kernel's activation staging, which is
 * how a decode step runs the q|k|v, FFN-up and logits projections (MT:469, 488, 906 followed by
 * MT:50-74).  Shapes whose rows do not fit the staging run the norm as a launch of its own.
 * h_dev [batch, k_in] f32; *fused_out (nullable) reports whether the folded form ran.
 * Unlike the other operators this call does more than enqueue: it allocates device memory for the
 * row statistics (or the normalised rows), with quantised weights it overwrites the weight's
 * activation staging buffer, and it synchronises `stream` before returning because those buffers
 * die with the call.  It must not be made on a stream that is being captured. */
int coeus_op_norm_gemv(const coeus_weight *w, const float *h_dev, uint64_t batch, uint32_t norm_kind,
                       const float *scale_dev, const float *bias_norm_dev, float eps, const float *bias_dev,
                       const float *residual_dev, uint32_t epilogue, float *y_dev, int *fused_out,
                       void *stream);
/* C[m, n_out] = epilogue(A[m, k_in] . W + bias) (+ residual): the prefill matmul. */
int coeus_op_gemm(const coeus_weight *w, const float *a_dev, uint64_t m, const float *bias_dev,
                  const float *residual_dev, uint32_t epilogue, float *c_dev, void *stream);
/* Measurement variant of coeus_op_gemm (no reference counterpart; used by the benchmark's
 * matrix-core roofline): runs the staging conversions and one untimed matmul, then launches the
 * matmul kernel `reps` times between two events on `stream` and returns the elapsed
 * milliseconds of those launches. */
int coeus_op_gemm_timed(const coeus_weight *w, const float *a_dev, uint64_t m, uint32_t epilogue,
                        float *c_dev, uint32_t reps, float *ms_out, void *stream);
/* One token id per row of logits_dev [rows, vocab] (device pointers; out_ids_dev uint64 [rows]).
 * `position` (the sequence position the token will take) and the row index key the random draw,
 * so a generation is reproducible from (seed, prompt).  GenerativeModel::generate's inner step
 * (CM:138-144); the reference has no sampler of its own, the rules are in sample.hip. */
int coeus_op_sample(const float *logits_dev, uint64_t rows, uint64_t vocab, const coeus_sampling *cfg,
                    uint64_t position, uint64_t *out_ids_dev, void *stream);
/* math::layer_norm (MT:105-128) over `rows` rows of `hidden`: scope COEUS_SCOPE_SEQUENCE uses
 * one mean/variance for the whole [rows*hidden] slice, COEUS_SCOPE_TOKEN one per row.
 * kind COEUS_NORM_RMSNORM ignores bias_dev. */
int coeus_op_norm(uint32_t kind, uint32_t scope, const float *x_dev, uint64_t rows, uint64_t hidden,
                  const float *scale_dev, const float *bias_dev, float eps, float *y_dev,
                  void *stream);
/* x[s, :] = E[ids[s], :] + PE[pos0 + s, :] (MT:812-835); ids_dev are uint64 on the device and
 * must already be range-checked; pe_dev is the sinusoidal table (MT:398-407). */
int coeus_op_embed(const float *table_dev, const float *pe_dev, const uint64_t *ids_dev,
                   uint64_t rows, uint64_t pos0, uint64_t hidden, float *x_dev, void *stream);
/* Causal multi-head attention (MT:219-278) on projected q,k,v: qkv_dev [rows, 3*inner] f32
 * holding q|k|v per row, out_dev [rows, inner]; scale 1/sqrt(head_dim) applied after the dot. */
int coeus_op_attention(const float *qkv_dev, uint64_t rows, uint64_t num_heads, uint64_t head_dim,
                       float *out_dev, void *stream);
/* The attention of ONE new token per sequence (the decode step's MT:219-278: the query row
 * against every cached key, row softmax, P.V) over a caller-owned 16-bit cache
 * [batch][num_heads][max_ctx][head_dim] (kv_dtype COEUS_KV_F16 or COEUS_KV_BF16; head_dim 64 or
 * 128) whose first `ctx` positions of every (sequence, head) hold keys / values.  qkv_dev
 * [batch, 3*inner] f32 as the q|k|v projection writes it (only the q third is read), out_dev
 * [batch, inner].  The context is split over `nsplit` workgroups per (sequence, head)
 * (flash-decoding; 0 = the library's choice for this shape, at most 32); their partial results
 * are merged by the last split to finish (merge = COEUS_MERGE_IN_KERNEL, what a decode step
 * runs) or by a second kernel (COEUS_MERGE_SEPARATE).  Synchronises `stream` before returning:
 * the partial-result buffer lives for this call. */
enum { COEUS_MERGE_IN_KERNEL = 0, COEUS_MERGE_SEPARATE = 1 };
int coeus_op_attention_decode(const float *qkv_dev, const void *k_cache_dev, const void *v_cache_dev,
                              uint32_t kv_dtype, uint64_t batch, uint64_t num_heads, uint64_t head_dim,
                              uint64_t max_ctx, uint64_t ctx, uint32_t nsplit, uint32_t merge,
                              float *out_dev, void *stream);
/* coeus_op_attention_decode for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same arguments and results; the partial records and arrival counters live in a
 * static device array of 2.04 MiB per GPU instead of a per-call allocation, so the call only
 * enqueues kernels on `stream` (no hipMalloc / hipFree, no synchronisation) and returns.  Limits:
 * batch * num_heads <= 1024 and batch * num_heads * nsplit <= 4096, COEUS_INVALID_INPUT beyond.
 * All calls on one GPU share the array: calls that overlap in time on one GPU (two streams, two
 * threads) race and must be serialised by the caller.  The first call on a device looks up the
 * array's address (once per device, no allocation); make that call outside a stream capture. */
int coeus_op_attention_decode_static(const float *qkv_dev, const void *k_cache_dev, const void *v_cache_dev,
                                     uint32_t kv_dtype, uint64_t batch, uint64_t num_heads,
                                     uint64_t head_dim, uint64_t max_ctx, uint64_t ctx, uint32_t nsplit,
                                     uint32_t merge, float *out_dev, void *stream);
/* Host-side sinusoidal table (MT:398-407), computed with the platform libm like the reference. */
int coeus_positional_encoding(uint64_t max_seq_len, uint64_t hidden_dim, float *table_out);

#ifdef __cplusplus
}
#endif
#endif /* COEUS_H */
