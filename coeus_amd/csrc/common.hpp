// Internal declarations shared by the translation units of libcoeus_mi355x.so.
// Target: gfx950 (MI355X, CDNA4) only; wavefront = 64 lanes.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "../../include/coeus.h"

namespace coeus {

// ---------------------------------------------------------------- errors
void set_error(const char *fmt, ...);
int fail(int status, const char *fmt, ...);

#define COEUS_HIP(expr)                                                                      \
    do {                                                                                     \
        hipError_t e_ = (expr);                                                              \
        if (e_ != hipSuccess)                                                                \
            return ::coeus::fail(e_ == hipErrorOutOfMemory ? COEUS_OUT_OF_MEMORY             \
                                                           : COEUS_DEVICE_ERROR,             \
                                 "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_),      \
                                 __FILE__, __LINE__);                                        \
    } while (0)

// Every extern "C" entry point runs between these: nothing is thrown across the boundary.
#define COEUS_GUARD_BEGIN try {
#define COEUS_GUARD_END                                                        \
    } catch (const std::bad_alloc &) {                                         \
        return fail(COEUS_OUT_OF_MEMORY, "host allocation failed");            \
    } catch (const std::exception &ex) {                                       \
        return fail(COEUS_DEVICE_ERROR, "unexpected failure: %s", ex.what());  \
    } catch (...) {                                                            \
        return fail(COEUS_DEVICE_ERROR, "unexpected failure");                 \
    }

#define COEUS_TRY(expr)                 \
    do {                                \
        int rc_ = (expr);               \
        if (rc_ != COEUS_OK) return rc_; \
    } while (0)

// ---------------------------------------------------------------- .rustllm files (rustllm_file.hip)
uint64_t rustllm_checksum(const float *params, uint64_t n);
int rustllm_write(const char *path, const coeus_config &cfg, const float *params, uint64_t n);
int rustllm_read_header(const char *path, coeus_config &cfg, uint64_t &n_params);
int rustllm_read_parameters(const char *path, float *params, uint64_t n);

// ---------------------------------------------------------------- small helpers
static inline uint64_t ceil_div(uint64_t a, uint64_t b) { return (a + b - 1) / b; }
static inline uint64_t round_up(uint64_t a, uint64_t b) { return ceil_div(a, b) * b; }

// ---------------------------------------------------------------- parameter layout
// Offsets into the flat f32 parameter buffer (MT:677-740 and the per-layer walk MT:839-880),
// generalised to a decoupled head_dim and a gated FFN.
struct Layout {
    uint64_t token_embed_offset, token_embed_size;
    uint64_t first_layer_offset, layer_stride;
    uint64_t ln1_scale, ln1_bias, wq, wk, wv, wo, bq, bk, bv, bo;
    uint64_t ln2_scale, ln2_bias, w_gate, w_up, w_down, b_gate, b_up, b_down;
    uint64_t final_ln_offset, output_proj_offset, output_proj_size;
    uint64_t used_params, total_params, inner_dim, head_dim;
};
Layout make_layout(const coeus_config &c);

// ---------------------------------------------------------------- device weights
// Linear weight W (reference layout [k_in, n_out]) resident on the device.
//   F32 / BF16 : row-major [n_out][k_in]  (each output's reduction run is contiguous)
//   Q8_0/Q4_0  : MFMA-native tiles.  Rows are grouped in tiles of 16, quantisation blocks in
//                groups of 4 (128 k).  One (tile, group) chunk stores, for lane = 16*g + r
//                (r = row in tile, g = 0..3), the 8 k-values 8g..8g+7 of blocks 4G..4G+3 of
//                row r: Q4_0 -> one dword per block (16 B per lane, 1 KiB per chunk),
//                Q8_0 -> two dwords per block (32 B per lane, stored as two 1 KiB halves).
//                A Q4_0 dword holds its 8 values at nibble positions [k0,k2,k4,k6,k1,k3,k5,k7].
//                Scales: f16 [tile][group][row=16][blk=4] (8 B per row and chunk).
struct Weight {
    uint32_t dtype = 0;
    uint64_t k = 0, n = 0;       // logical sizes
    uint64_t k_pad = 0, n_pad = 0; // padded to 128 / 16 for quantised types
    void *data = nullptr;        // weights (quants for Q*)
    __half *scales = nullptr;    // Q* only
    uint64_t bytes = 0;
    __half *xq_scratch = nullptr; // [k_pad/8][16][8] f16 staging for the operator-level API
    // Q* only: dense f16 copy [n] rows of gemm_ld(k) elements for the prefill matmul, made on first
    // use and kept while the owner's budget lasts (7B: 13.7 GB next to 4.2 GB of quants; the card
    // has 288 GB).  Saves re-expanding every weight on every prompt pass.
    mutable __half *expanded = nullptr;
};
int weight_alloc(Weight &w, uint32_t dtype, uint64_t k, uint64_t n);
void weight_free(Weight &w);

// Where a device weight's values come from.  Output column j of the packed weight is taken from
// one of several consecutive [k, n_part] matrices of the flat parameter buffer:
//   interleave == 0: part = j / n_part, column j % n_part   (Wq|Wk|Wv fused into one matmul)
//   interleave == 1: part = j % 2,      column j / 2        (gate_m, up_m on adjacent rows)
// Element (l, j) has flat index base + part*k*n_part + l*n_part + column.  With `params` set
// the value is params[index]; otherwise it is 0.02 * z(seed, index).
struct WeightSource {
    const float *params = nullptr;  // device pointer (may be offset so that `base` is absolute)
    uint64_t seed = 0;
    uint64_t base = 0;
    uint64_t n_part = 0;
    uint32_t interleave = 0;
};
int weight_pack(Weight &w, const WeightSource &src, hipStream_t st);
// Q* only: makes the resident f16 copy for the prefill matmul (Weight::expanded) if `budget`
// still covers it, and charges the budget; does nothing for other types or when it does not fit.
int weight_expand(const Weight &w, uint64_t *budget, hipStream_t st);
int weight_unpack_to_device(const Weight &w, float *dst_kn, hipStream_t st);

// Host/device counter-based generator (see weights.hip).
float synth_value_host(uint64_t seed, uint64_t index);  // 0.02 * z(seed, index)
int launch_fill_seeded(float *dst, uint64_t n, uint64_t seed, uint64_t base, float mean,
                       hipStream_t st);
// Row stride (elements) of the 16-bit staging matrices of the prefill matmul.  Rows that lie a
// power of two apart would send a tile's 256 row slices to the same few memory channels; one
// extra 128-byte line per row rotates them over all channels.
static inline uint64_t gemm_ld(uint64_t k) { return k + 64; }
// [rows][k] f32 -> 16-bit (bf16 or f16) rows of stride ld
int launch_f32_to_16(const float *src, void *dst, uint64_t rows, uint64_t k, uint64_t ld, bool bf16,
                     hipStream_t st);
int launch_f32_to_bf16(const float *src, uint16_t *dst, uint64_t n, hipStream_t st);
// Dequantise a Q8_0/Q4_0 weight into a dense f16 matrix [n] rows of stride ld (value = f16(q * d)).
int launch_dequant_to_f16(const Weight &w, __half *dst_nk, uint64_t ld, hipStream_t st);

// ---------------------------------------------------------------- kernels (launchers)
// Activation interchange format for the quantised decode matmul ("xq"): f16,
// [k_pad/8][bp][8] where bp = padded batch (1,2,4,8,16): element (b, k) sits at
// ((k/8)*bp + b)*8 + k%8.  Padding positions hold zeros.
static inline uint32_t pad_batch(uint64_t b) { return b <= 1 ? 1 : b <= 2 ? 2 : b <= 4 ? 4 : b <= 8 ? 8 : 16; }

int launch_pack_xq(const float *x, uint64_t batch, uint64_t k, uint64_t k_pad, __half *xq,
                   hipStream_t st);

// 16-bit output rows for the next prefill matmul's A operand (bf16 or f16, row stride ld elements):
// producers write them directly so no separate conversion pass reads the f32 result back.
struct LpOut {
    void *p = nullptr;
    uint64_t ld = 0;
    bool bf16 = false;
};

struct Epilogue {
    const float *bias = nullptr;     // [n]
    const float *residual = nullptr; // [rows, n_eff]
    uint32_t act = COEUS_EPI_NONE;   // COEUS_EPI_*
    float *out_f32 = nullptr;        // [rows, n_eff] (nullable if out_xq set)
    __half *out_xq = nullptr;        // xq format with bp_out (decode chaining)
    uint32_t bp_out = 0;
    // decode q|k|v projection: write the k and v thirds into the cache at position *kv_pos
    void *kv_k = nullptr, *kv_v = nullptr;
    const uint32_t *kv_pos = nullptr;
    uint32_t kv_dtype = 0, kv_inner = 0, kv_heads = 0, kv_hd = 0, kv_max_ctx = 0;
    // prompt pass (launch_gemm, where gemm_appends_kv says so): rows are kv_rows_per_seq tokens per
    // sequence, token i of a sequence goes to cache position kv_pos0 + i; kv_pos is not used
    uint32_t kv_rows_per_seq = 0, kv_pos0 = 0;
    // decode matmuls that produce the residual stream: per-(row, 16 outputs) {sum, M2} records
    // [rows][ceil(n/16)] for the norm folded into the next matmul (see NormFuse::stats)
    float2 *stats_out = nullptr;
    // ... and, for a root-mean-square norm, the stored values times that norm's scale (NormFuse::g):
    // g_out[row * n + j] = value * g_scale[j].  Batches of up to 4 (gemv_quad_kernel) only.
    const float *g_scale = nullptr;
    float *g_out = nullptr;
    LpOut out_lp;                    // prefill matmul: 16-bit copy of the output (out_f32 nullable then)
};

// Normalisation folded into the decode matmul's activation staging: x = norm(h) row by row.
struct NormFuse {
    const float *h = nullptr;      // [batch, k] f32 residual stream
    const float *scale = nullptr;  // [k]
    const float *bias = nullptr;   // [k] (LayerNorm only)
    float eps = 0.f;
    uint32_t kind = COEUS_NORM_LAYERNORM;
    // [batch][ceil(k/16)] {sum, M2} records of h written by its producer (Epilogue::stats_out or
    // launch_embed): the row statistics are merged from them instead of being reduced again by
    // every workgroup
    const float2 *stats = nullptr;
    // RMSNorm only (nullable): h * scale [batch, k] f32, written by the producer of h next to the
    // records (Epilogue::g_out, launch_embed).  The consuming matmul then stages half the bytes
    // (16 KB instead of 32 KB per workgroup at k = 4096) and multiplies by 1 / rms.
    const float *g = nullptr;
};
// True when launch_gemv can take `nf` for this weight and batch (quantised weights whose whole
// activation block fits in LDS).
bool gemv_can_fuse_norm(const Weight &w, uint64_t batch);
// The same for f32 / bf16 weights (the normalised block [batch, k] f32 has to fit in LDS; the
// statistics are computed inside the launch, NormFuse::stats is not used).
bool gemv_can_fuse_norm_dense(const Weight &w, uint64_t batch);
// The same normalisation as a launch of its own (batches too large for the folded form):
// nf.h rows -> xq, row statistics merged from nf.stats.  Padding rows of xq are not written.
int launch_norm_from_stats(const NormFuse &nf, uint64_t batch, uint64_t k, uint64_t k_pad, __half *xq,
                           hipStream_t st);

// {sum, M2} records of every 16 consecutive elements of each row of h [rows, k] -> stats
// [rows][ceil(k/16)] (NormFuse::stats for rows that no matmul epilogue produced).
int launch_row_stats16(const float *h, uint64_t rows, uint64_t k, float2 *stats, hipStream_t st);

// Decode matmul: rows = batch <= 16.  x is f32 [batch, k] for F32/BF16 weights and xq for
// quantised weights.
int launch_gemv(const Weight &w, const void *x, uint64_t batch, const Epilogue &ep, hipStream_t st,
                const NormFuse *nf = nullptr);

// Prefill matmul on f32 activations: C[m, n] = A[m, k] . W.  Low-precision weights need
// staging: a_lp holds A rounded to the matrix-core input type ([m, k] 16-bit), w_lp a dense
// f16 copy of a quantised weight ([n, k]).
struct GemmScratch {
    void *a_lp = nullptr;
    uint64_t a_lp_bytes = 0;
    void *w_lp = nullptr;
    uint64_t w_lp_bytes = 0;
    // measurement: launch the matrix-core kernel `repeat` times between two events (the staging
    // conversions run once, before the first event)
    uint32_t repeat = 1;
    hipEvent_t ev_begin = nullptr, ev_end = nullptr;
    // bytes that may still be spent on resident expanded copies of quantised weights (nullable:
    // no resident copies, every call expands into w_lp)
    uint64_t *expand_budget = nullptr;
    // room for the partial products of a k-split launch (nullable: no splitting)
    float *partials = nullptr;
    uint64_t partials_bytes = 0;
};
// Bytes of GemmScratch::partials that launch_gemm would use for this weight on m rows (0: it would
// not split).
uint64_t gemm_split_scratch_bytes(const Weight &w, uint64_t m);
// Short prompts on quantised weights: the matmul that streams the quantised blocks (gemv.hip).
struct EpiArgs;
bool gemm_uses_qskinny(const Weight &w, uint64_t m);
uint64_t gemm_qskinny_scratch_bytes(const Weight &w, uint64_t m);
int launch_gemm_qskinny(const Weight &w, const uint16_t *a, uint64_t lda, uint64_t m, const EpiArgs &e,
                        float *partials, uint64_t partials_bytes, uint32_t *splits_out, hipStream_t st);
// a_staged: `a` already is the 16-bit staged matrix (rows of gemm_ld(k) elements, the weight's
// matrix-core input type), written by the producer through an LpOut.
// True when launch_gemm's kernel for this weight and row count can write the key and value
// thirds of a q|k|v projection straight into the cache (Epilogue::kv_* with kv_rows_per_seq).
bool gemm_appends_kv(const Weight &w, uint64_t m, uint64_t inner, uint64_t hd);
int launch_gemm(const Weight &w, const void *a, uint64_t m, const Epilogue &ep, GemmScratch &scr,
                hipStream_t st, bool a_staged = false);

// `partials` (nullable; norm_sequence_scratch_bytes() of device memory, used by whole-slice
// statistics only): lets a large slice be reduced by many workgroups instead of one.
int launch_norm(uint32_t kind, uint32_t scope, const float *x, uint64_t rows, uint64_t hidden,
                const float *scale, const float *bias, float eps, float *y, __half *y_xq,
                uint32_t bp, hipStream_t st, const LpOut *y_lp = nullptr, double *partials = nullptr);
size_t norm_sequence_scratch_bytes();
int launch_embed(const void *table, bool table_bf16, const float *pe, const uint64_t *ids,
                 uint64_t rows, uint64_t rows_per_seq, uint64_t pos0, const uint32_t *pos_dev,
                 uint64_t hidden, float *x, float2 *stats, hipStream_t st, const float *g_scale = nullptr,
                 float *g_out = nullptr);
// g[row][k] = h[row][k] * scale[k] (NormFuse::g for rows that no epilogue produced)
int launch_prescale(const float *h, const float *scale, uint64_t rows, uint64_t k, float *g, hipStream_t st);
// `advance` (nullable; rows == 1 only): {position, step} counters that the kernel increments
// after storing its result, which saves the launch_advance that would follow.
int launch_argmax(const float *logits, uint64_t rows, uint64_t vocab, uint64_t *out_ids,
                  uint64_t *history, uint64_t history_stride, const uint32_t *step_dev,
                  hipStream_t st, uint32_t *advance = nullptr);
int launch_advance(uint32_t *pos, uint32_t *step, hipStream_t st);
int launch_sample(const float *logits, uint64_t rows, uint64_t vocab, const coeus_sampling &cfg,
                  uint64_t pos0, const uint32_t *pos_dev, uint64_t *out_ids, uint64_t *history,
                  uint64_t history_stride, const uint32_t *step_dev, hipStream_t st);

int launch_kv_append(const float *qkv, void *kc, void *vc, uint32_t kv_dtype, uint64_t batch,
                     uint64_t n, uint64_t heads, uint64_t hd, uint64_t max_ctx, uint64_t pos0,
                     const uint32_t *pos_dev, hipStream_t st);
uint32_t attn_decode_splits(uint64_t batch, uint64_t heads, uint64_t max_ctx);
// True when n new rows per sequence take the matrix-core prefill kernel (which can write 16-bit
// output rows) rather than the generic one.
bool attn_prefill_on_matrix_cores(uint64_t n, uint64_t hd, uint32_t kv_dtype);
// Attention of n new rows per sequence (positions pos..pos+n-1) against the cache.
// part_scratch: [batch*heads*nsplit*(head_dim+2)] f32 for the split decode kernel (nullable);
// counters: [batch*heads] zeroed u32 -> the last split merges in-kernel (else a merge kernel runs).
int launch_attention(const float *qkv, const void *kc, const void *vc, uint32_t kv_dtype,
                     uint64_t batch, uint64_t n, uint64_t heads, uint64_t hd, uint64_t max_ctx,
                     uint64_t pos0, const uint32_t *pos_dev, float *out, __half *out_xq,
                     uint32_t bp, float *part_scratch, uint32_t nsplit, uint32_t *counters,
                     hipStream_t st, const LpOut *out_lp = nullptr);

}  // namespace coeus
