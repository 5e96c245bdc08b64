// extern "C" surface of libcoeus_mi355x.so (declared in include/coeus.h).  Nothing here throws
// across the boundary: every entry point catches and reports through coeus_last_error().
#include <cmath>
#include <new>

#include "model.hpp"

using namespace coeus;

struct coeus_weight { Weight w; };

extern "C" {

int coeus_device_info(char *name_out, uint64_t name_cap, uint64_t *hbm_bytes, uint32_t *compute_units) {
    COEUS_GUARD_BEGIN
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n == 0)
        return fail(COEUS_DEVICE_ERROR, "no HIP device visible");
    hipDeviceProp_t p;
    COEUS_HIP(hipGetDeviceProperties(&p, 0));
    if (name_out && name_cap) snprintf(name_out, name_cap, "%s (%s)", p.name, p.gcnArchName);
    if (hbm_bytes) *hbm_bytes = p.totalGlobalMem;
    if (compute_units) *compute_units = (uint32_t)p.multiProcessorCount;
    return COEUS_OK;
    COEUS_GUARD_END
}

// ---------------------------------------------------------------- device plumbing
int coeus_device_malloc(uint64_t bytes, void **out) {
    if (!out) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    *out = nullptr;
    COEUS_HIP(hipMalloc(out, bytes ? bytes : 1));
    return COEUS_OK;
}
int coeus_device_free(void *ptr) {
    if (ptr) COEUS_HIP(hipFree(ptr));
    return COEUS_OK;
}
int coeus_memcpy_h2d(void *dst, const void *src, uint64_t bytes) {
    if (bytes) COEUS_HIP(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
    return COEUS_OK;
}
int coeus_memcpy_d2h(void *dst, const void *src, uint64_t bytes) {
    if (bytes) COEUS_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
    return COEUS_OK;
}
int coeus_device_memset(void *dst, int value, uint64_t bytes) {
    if (bytes) COEUS_HIP(hipMemset(dst, value, bytes));
    return COEUS_OK;
}
namespace coeus {
__global__ __launch_bounds__(256) void device_copy_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, uint64_t n16) {
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (uint64_t)gridDim.x * blockDim.x)
        dst[i] = src[i];
}
}  // namespace coeus
int coeus_device_copy(void *dst, const void *src, uint64_t bytes, void *stream) {
    if (!dst || !src) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    if (bytes % 16) return fail(COEUS_INVALID_INPUT, "copy size %llu is not a multiple of 16", (unsigned long long)bytes);
    if (bytes == 0) return COEUS_OK;
    const uint64_t n16 = bytes / 16;
    const unsigned grid = (unsigned)(n16 / 256 < 8192 ? (n16 + 255) / 256 : 8192);
    hipLaunchKernelGGL(coeus::device_copy_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, (const uint4 *)src, (uint4 *)dst, n16);
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}
int coeus_device_synchronize(void) {
    COEUS_HIP(hipDeviceSynchronize());
    return COEUS_OK;
}
int coeus_stream_create(void **out) {
    if (!out) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    hipStream_t s = nullptr;
    COEUS_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *out = s;
    return COEUS_OK;
}
int coeus_stream_synchronize(void *stream) {
    COEUS_HIP(hipStreamSynchronize((hipStream_t)stream));
    return COEUS_OK;
}
int coeus_stream_destroy(void *stream) {
    if (stream) COEUS_HIP(hipStreamDestroy((hipStream_t)stream));
    return COEUS_OK;
}
int coeus_event_create(void **out) {
    if (!out) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    hipEvent_t e = nullptr;
    COEUS_HIP(hipEventCreate(&e));
    *out = e;
    return COEUS_OK;
}
int coeus_event_record(void *event, void *stream) {
    COEUS_HIP(hipEventRecord((hipEvent_t)event, (hipStream_t)stream));
    return COEUS_OK;
}
int coeus_event_synchronize(void *event) {
    COEUS_HIP(hipEventSynchronize((hipEvent_t)event));
    return COEUS_OK;
}
int coeus_event_elapsed_ms(void *start, void *stop, float *ms_out) {
    if (!ms_out) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    COEUS_HIP(hipEventElapsedTime(ms_out, (hipEvent_t)start, (hipEvent_t)stop));
    return COEUS_OK;
}
int coeus_event_destroy(void *event) {
    if (event) COEUS_HIP(hipEventDestroy((hipEvent_t)event));
    return COEUS_OK;
}

// ---------------------------------------------------------------- model
static int create_common(const coeus_config *cfg, const float *params, uint64_t n, uint64_t seed,
                         coeus_model **out) {
    COEUS_GUARD_BEGIN
    if (!cfg || !out) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    *out = nullptr;
    Model *m = nullptr;
    COEUS_TRY(model_create(*cfg, params, n, seed, &m));
    *out = reinterpret_cast<coeus_model *>(m);
    return COEUS_OK;
    COEUS_GUARD_END
}

int coeus_model_create(const coeus_config *cfg, const float *params, uint64_t n_params, coeus_model **out) {
    if (!params) return fail(COEUS_INVALID_INPUT, "null parameter buffer");
    return create_common(cfg, params, n_params, 0, out);
}

int coeus_model_create_seeded(const coeus_config *cfg, uint64_t seed, coeus_model **out) {
    return create_common(cfg, nullptr, 0, seed, out);
}

static Model *M(coeus_model *m) { return reinterpret_cast<Model *>(m); }
static const Model *M(const coeus_model *m) { return reinterpret_cast<const Model *>(m); }
static Session *S(coeus_session *s) { return reinterpret_cast<Session *>(s); }

int coeus_model_forward(coeus_model *m, const uint64_t *ids, uint64_t seq_len, float *logits_out) {
    COEUS_GUARD_BEGIN
    if (!m) return fail(COEUS_INVALID_INPUT, "null model");
    return model_forward(*M(m), ids, seq_len, logits_out, false);
    COEUS_GUARD_END
}

int coeus_model_forward_all(coeus_model *m, const uint64_t *ids, uint64_t seq_len, float *logits_out) {
    COEUS_GUARD_BEGIN
    if (!m) return fail(COEUS_INVALID_INPUT, "null model");
    return model_forward(*M(m), ids, seq_len, logits_out, true);
    COEUS_GUARD_END
}

uint64_t coeus_model_num_parameters(const coeus_model *m) { return m ? M(m)->n_params : 0; }
const coeus_config *coeus_model_config(const coeus_model *m) { return m ? &M(m)->cfg : nullptr; }
const char *coeus_model_name(const coeus_model *m) { (void)m; return "TransformerModel"; }  // MT:782-784
uint64_t coeus_model_weight_bytes(const coeus_model *m) { return m ? M(m)->weight_bytes : 0; }
uint64_t coeus_model_resident_bytes(const coeus_model *m) {
    if (!m) return 0;
    Model *mm = const_cast<Model *>(M(m));
    std::lock_guard<std::mutex> lock(mm->mu);  // prompt passes charge the budget under this lock
    return mm->weight_bytes + (Model::kExpandBudget - mm->expand_budget);
}
void coeus_model_destroy(coeus_model *m) { delete M(m); }

// ---------------------------------------------------------------- sessions
int coeus_session_create(coeus_model *m, uint64_t batch, uint64_t max_ctx, coeus_session **out) {
    COEUS_GUARD_BEGIN
    if (!m || !out) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    *out = nullptr;
    Session *s = nullptr;
    COEUS_TRY(session_create(*M(m), batch, max_ctx, &s));
    *out = reinterpret_cast<coeus_session *>(s);
    return COEUS_OK;
    COEUS_GUARD_END
}

int coeus_session_prefill(coeus_session *s, const uint64_t *ids, uint64_t n, float *logits_out) {
    COEUS_GUARD_BEGIN
    if (!s) return fail(COEUS_INVALID_INPUT, "null session");
    return session_prefill(*S(s), ids, n, logits_out);
    COEUS_GUARD_END
}

int coeus_session_decode(coeus_session *s, const uint64_t *ids, float *logits_out) {
    COEUS_GUARD_BEGIN
    if (!s) return fail(COEUS_INVALID_INPUT, "null session");
    return session_decode(*S(s), ids, logits_out);
    COEUS_GUARD_END
}

int coeus_session_decode_greedy(coeus_session *s, const uint64_t *first_ids, uint64_t n_steps,
                                uint64_t *out_ids) {
    COEUS_GUARD_BEGIN
    if (!s) return fail(COEUS_INVALID_INPUT, "null session");
    return session_decode_greedy(*S(s), first_ids, n_steps, out_ids);
    COEUS_GUARD_END
}

int coeus_session_generate(coeus_session *s, const uint64_t *first_ids, uint64_t n_steps,
                           const coeus_sampling *cfg, uint64_t *out_ids) {
    COEUS_GUARD_BEGIN
    if (!s) return fail(COEUS_INVALID_INPUT, "null session");
    return session_decode_greedy(*S(s), first_ids, n_steps, out_ids, cfg);
    COEUS_GUARD_END
}

int coeus_op_sample(const float *logits_dev, uint64_t rows, uint64_t vocab, const coeus_sampling *cfg,
                    uint64_t position, uint64_t *out_ids_dev, void *stream) {
    COEUS_GUARD_BEGIN
    if (!logits_dev || !cfg || !out_ids_dev) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    return launch_sample(logits_dev, rows, vocab, *cfg, position, nullptr, out_ids_dev, nullptr, 0, nullptr,
                         (hipStream_t)stream);
    COEUS_GUARD_END
}

int coeus_session_time_decode_matmuls(coeus_session *s, uint64_t reps, float *ms_out,
                                      uint64_t *launches_out, uint64_t *bytes_out) {
    COEUS_GUARD_BEGIN
    if (!s) return fail(COEUS_INVALID_INPUT, "null session");
    return session_time_decode_matmuls(*S(s), reps, ms_out, launches_out, bytes_out);
    COEUS_GUARD_END
}

int coeus_session_time_decode_attention(coeus_session *s, uint64_t reps, float *ms_out,
                                        uint64_t *launches_out, uint64_t *bytes_out) {
    COEUS_GUARD_BEGIN
    if (!s) return fail(COEUS_INVALID_INPUT, "null session");
    return session_time_decode_attention(*S(s), reps, ms_out, launches_out, bytes_out);
    COEUS_GUARD_END
}

int coeus_session_set_graph(coeus_session *s, int enabled) {
    if (!s) return fail(COEUS_INVALID_INPUT, "null session");
    if (enabled)
        if (const char *why = graph_replay_forbidden())
            return fail(COEUS_INVALID_INPUT, "graph replay refused: %s", why);
    std::lock_guard<std::mutex> lock(S(s)->m->mu);
    S(s)->use_graph = enabled != 0;
    return COEUS_OK;
}

int coeus_session_graph_enabled(const coeus_session *s) {
    if (!s) return 0;
    const Session *ss = reinterpret_cast<const Session *>(s);
    std::lock_guard<std::mutex> lock(ss->m->mu);
    return ss->use_graph ? 1 : 0;
}

uint64_t coeus_session_position(const coeus_session *s) {
    if (!s) return 0;
    const Session *ss = reinterpret_cast<const Session *>(s);
    std::lock_guard<std::mutex> lock(ss->m->mu);
    return ss->pos;
}

int coeus_session_reset(coeus_session *s) {
    if (!s) return fail(COEUS_INVALID_INPUT, "null session");
    std::lock_guard<std::mutex> lock(S(s)->m->mu);
    S(s)->pos = 0;
    return COEUS_OK;
}

void coeus_session_destroy(coeus_session *s) { delete S(s); }

// ---------------------------------------------------------------- operators
static int weight_create_common(uint32_t dtype, const float *host_w, uint64_t seed, uint64_t base,
                                uint64_t k, uint64_t n, coeus_weight **out) {
    COEUS_GUARD_BEGIN
    if (!out) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    *out = nullptr;
    std::unique_ptr<coeus_weight> w(new coeus_weight());
    int rc = weight_alloc(w->w, dtype, k, n);
    if (rc != COEUS_OK) { weight_free(w->w); return rc; }
    float *dev = nullptr;
    WeightSource src;
    src.seed = seed;
    src.base = base;
    src.n_part = n;
    if (host_w) {
        hipError_t e = hipMalloc((void **)&dev, k * n * 4);
        if (e == hipSuccess) e = hipMemcpy(dev, host_w, k * n * 4, hipMemcpyHostToDevice);
        if (e != hipSuccess) {
            if (dev) (void)hipFree(dev);
            weight_free(w->w);
            return fail(COEUS_DEVICE_ERROR, "weight upload failed: %s", hipGetErrorString(e));
        }
        src.params = dev;
        src.base = 0;
    }
    rc = weight_pack(w->w, src, nullptr);
    hipError_t e = hipDeviceSynchronize();
    if (dev) (void)hipFree(dev);
    if (rc == COEUS_OK && e != hipSuccess) rc = fail(COEUS_DEVICE_ERROR, "weight packing failed: %s", hipGetErrorString(e));
    if (rc == COEUS_OK && dtype >= COEUS_W_Q8_0) {
        e = hipMalloc((void **)&w->w.xq_scratch, w->w.k_pad * 16 * 2);
        if (e != hipSuccess) rc = fail(COEUS_OUT_OF_MEMORY, "hipMalloc(xq scratch) failed");
    }
    if (rc != COEUS_OK) { weight_free(w->w); return rc; }
    *out = w.release();
    return COEUS_OK;
    COEUS_GUARD_END
}

int coeus_weight_create(uint32_t dtype, const float *host_w, uint64_t k_in, uint64_t n_out, coeus_weight **out) {
    if (!host_w) return fail(COEUS_INVALID_INPUT, "null weight matrix");
    return weight_create_common(dtype, host_w, 0, 0, k_in, n_out, out);
}

int coeus_weight_create_seeded(uint32_t dtype, uint64_t seed, uint64_t base_index, uint64_t k_in,
                               uint64_t n_out, coeus_weight **out) {
    return weight_create_common(dtype, nullptr, seed, base_index, k_in, n_out, out);
}

int coeus_weight_dequantize(const coeus_weight *w, float *host_out) {
    COEUS_GUARD_BEGIN
    if (!w || !host_out) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    float *dev = nullptr;
    const uint64_t bytes = w->w.k * w->w.n * 4;
    COEUS_HIP(hipMalloc((void **)&dev, bytes));
    int rc = weight_unpack_to_device(w->w, dev, nullptr);
    hipError_t e = rc == COEUS_OK ? hipMemcpy(host_out, dev, bytes, hipMemcpyDeviceToHost) : hipSuccess;
    (void)hipFree(dev);
    if (rc != COEUS_OK) return rc;
    COEUS_HIP(e);
    return COEUS_OK;
    COEUS_GUARD_END
}

uint64_t coeus_weight_bytes(const coeus_weight *w) { return w ? w->w.bytes : 0; }

void coeus_weight_destroy(coeus_weight *w) {
    if (!w) return;
    weight_free(w->w);
    delete w;
}

static Epilogue make_user_epilogue(const float *bias, const float *residual, uint32_t epilogue, float *y) {
    Epilogue e;
    e.bias = bias;
    e.residual = residual;
    e.act = epilogue;
    e.out_f32 = y;
    return e;
}

int coeus_op_gemv(const coeus_weight *w, const float *x_dev, uint64_t batch, const float *bias_dev,
                  const float *residual_dev, uint32_t epilogue, float *y_dev, void *stream) {
    COEUS_GUARD_BEGIN
    if (!w || !x_dev || !y_dev) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    if (epilogue > COEUS_EPI_SILU_GATE) return fail(COEUS_INVALID_INPUT, "unknown epilogue %u", epilogue);
    if (batch == 0 || batch > 16)
        return fail(COEUS_INVALID_INPUT, "decode matmul batch %llu out of range [1, 16]", (unsigned long long)batch);
    hipStream_t st = (hipStream_t)stream;
    const Epilogue e = make_user_epilogue(bias_dev, residual_dev, epilogue, y_dev);
    if (w->w.dtype >= COEUS_W_Q8_0) {
        // f32 activations are rounded to f16 in the kernel's interchange format first
        COEUS_TRY(launch_pack_xq(x_dev, batch, w->w.k, w->w.k_pad, w->w.xq_scratch, st));
        return launch_gemv(w->w, w->w.xq_scratch, batch, e, st);
    }
    return launch_gemv(w->w, x_dev, batch, e, st);
    COEUS_GUARD_END
}

int coeus_op_norm_gemv(const coeus_weight *w, const float *h_dev, uint64_t batch, uint32_t norm_kind,
                       const float *scale_dev, const float *bias_norm_dev, float eps, const float *bias_dev,
                       const float *residual_dev, uint32_t epilogue, float *y_dev, int *fused_out,
                       void *stream) {
    COEUS_GUARD_BEGIN
    if (!w || !h_dev || !y_dev || !scale_dev || (norm_kind == COEUS_NORM_LAYERNORM && !bias_norm_dev))
        return fail(COEUS_INVALID_INPUT, "null pointer argument");
    if (norm_kind > COEUS_NORM_RMSNORM) return fail(COEUS_INVALID_INPUT, "unknown norm kind %u", norm_kind);
    if (epilogue > COEUS_EPI_SILU_GATE) return fail(COEUS_INVALID_INPUT, "unknown epilogue %u", epilogue);
    if (batch == 0 || batch > 16)
        return fail(COEUS_INVALID_INPUT, "decode matmul batch %llu out of range [1, 16]", (unsigned long long)batch);
    hipStream_t st = (hipStream_t)stream;
    const Weight &W = w->w;
    const Epilogue e = make_user_epilogue(bias_dev, residual_dev, epilogue, y_dev);
    NormFuse nf;
    nf.h = h_dev; nf.scale = scale_dev; nf.bias = bias_norm_dev; nf.eps = eps; nf.kind = norm_kind;
    const bool quant = W.dtype >= COEUS_W_Q8_0;
    const bool fused = quant ? gemv_can_fuse_norm(W, batch) : gemv_can_fuse_norm_dense(W, batch);
    if (fused_out) *fused_out = fused ? 1 : 0;
    DeviceBuf stats, x;
    int rc = COEUS_OK;
    if (quant && fused) {
        rc = stats.ensure(batch * ceil_div(W.k, 16) * sizeof(float2));
        if (rc == COEUS_OK) rc = launch_row_stats16(h_dev, batch, W.k, (float2 *)stats.p, st);
        nf.stats = (const float2 *)stats.p;
        if (rc == COEUS_OK && norm_kind == COEUS_NORM_RMSNORM) {
            // as a decode step runs it: the rows arrive as h * scale, what the producer of h would have
            // stored next to the records
            rc = x.ensure(batch * W.k * 4);
            if (rc == COEUS_OK) rc = launch_prescale(h_dev, scale_dev, batch, W.k, (float *)x.p, st);
            nf.g = (const float *)x.p;
        }
        if (rc == COEUS_OK) rc = launch_gemv(W, nullptr, batch, e, st, &nf);
    } else if (fused) {
        rc = launch_gemv(W, nullptr, batch, e, st, &nf);
    } else if (quant) {
        // norm as its own launch, straight into the matmul's f16 interchange format (padding rows
        // and columns of the staging buffer are cleared first)
        const uint32_t bp = pad_batch(batch);
        hipError_t me = hipMemsetAsync(W.xq_scratch, 0, W.k_pad * 16 * 2, st);
        if (me != hipSuccess) rc = fail(COEUS_DEVICE_ERROR, "hipMemsetAsync failed: %s", hipGetErrorString(me));
        if (rc == COEUS_OK && (W.k & 7) == 0) {
            // as a decode step does it: row statistics merged from the per-16 records
            rc = stats.ensure(batch * ceil_div(W.k, 16) * sizeof(float2));
            if (rc == COEUS_OK) rc = launch_row_stats16(h_dev, batch, W.k, (float2 *)stats.p, st);
            nf.stats = (const float2 *)stats.p;
            if (rc == COEUS_OK) rc = launch_norm_from_stats(nf, batch, W.k, W.k_pad, W.xq_scratch, st);
        } else if (rc == COEUS_OK) {
            rc = launch_norm(norm_kind, COEUS_SCOPE_TOKEN, h_dev, batch, W.k, scale_dev, bias_norm_dev, eps, nullptr,
                             W.xq_scratch, bp, st);
        }
        if (rc == COEUS_OK) rc = launch_gemv(W, W.xq_scratch, batch, e, st);
    } else {
        rc = x.ensure(batch * W.k * 4);
        if (rc == COEUS_OK)
            rc = launch_norm(norm_kind, COEUS_SCOPE_TOKEN, h_dev, batch, W.k, scale_dev, bias_norm_dev, eps,
                             (float *)x.p, nullptr, 0, st);
        if (rc == COEUS_OK) rc = launch_gemv(W, x.p, batch, e, st);
    }
    if (stats.p || x.p) {  // the buffers die with this call: wait for the kernels that read them
        hipError_t se = hipStreamSynchronize(st);
        stats.release();
        x.release();
        if (rc == COEUS_OK && se != hipSuccess) rc = fail(COEUS_DEVICE_ERROR, "matmul failed: %s", hipGetErrorString(se));
    }
    return rc;
    COEUS_GUARD_END
}

int coeus_op_gemm(const coeus_weight *w, const float *a_dev, uint64_t m, const float *bias_dev,
                  const float *residual_dev, uint32_t epilogue, float *c_dev, void *stream) {
    COEUS_GUARD_BEGIN
    if (!w || !a_dev || !c_dev) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    if (epilogue > COEUS_EPI_SILU_GATE) return fail(COEUS_INVALID_INPUT, "unknown epilogue %u", epilogue);
    hipStream_t st = (hipStream_t)stream;
    const Epilogue e = make_user_epilogue(bias_dev, residual_dev, epilogue, c_dev);
    GemmScratch scr;
    DeviceBuf a_lp, w_lp, part;
    if (w->w.dtype != COEUS_W_F32) {
        COEUS_TRY(a_lp.ensure(m * gemm_ld(w->w.k) * 2));
        if (w->w.dtype >= COEUS_W_Q8_0) {
            int rc = w_lp.ensure(w->w.n * gemm_ld(w->w.k) * 2);
            if (rc != COEUS_OK) { a_lp.release(); return rc; }
        }
        scr.a_lp = a_lp.p; scr.a_lp_bytes = a_lp.bytes;
        scr.w_lp = w_lp.p; scr.w_lp_bytes = w_lp.bytes;
    }
    // (a launch of few tiles is split along k when it has room for the partial products; without
    // the room it runs unsplit)
    if (const uint64_t pb = gemm_split_scratch_bytes(w->w, m))
        if (part.ensure(pb) != COEUS_OK) part.release();
    scr.partials = (float *)part.p; scr.partials_bytes = part.bytes;
    int rc = launch_gemm(w->w, a_dev, m, e, scr, st);
    if (a_lp.p || w_lp.p || part.p) {
        // the staging buffers die with this call: wait for the kernels that read them
        hipError_t se = hipStreamSynchronize(st);
        a_lp.release();
        w_lp.release();
        part.release();
        if (rc == COEUS_OK && se != hipSuccess) rc = fail(COEUS_DEVICE_ERROR, "matmul failed: %s", hipGetErrorString(se));
    }
    return rc;
    COEUS_GUARD_END
}

int coeus_op_gemm_timed(const coeus_weight *w, const float *a_dev, uint64_t m, uint32_t epilogue,
                        float *c_dev, uint32_t reps, float *ms_out, void *stream) {
    COEUS_GUARD_BEGIN
    if (!w || !a_dev || !c_dev || !ms_out || reps == 0) return fail(COEUS_INVALID_INPUT, "bad timing arguments");
    if (epilogue > COEUS_EPI_SILU_GATE) return fail(COEUS_INVALID_INPUT, "unknown epilogue %u", epilogue);
    hipStream_t st = (hipStream_t)stream;
    const Epilogue e = make_user_epilogue(nullptr, nullptr, epilogue, c_dev);
    GemmScratch scr;
    DeviceBuf a_lp, w_lp, part;
    if (w->w.dtype != COEUS_W_F32) {
        COEUS_TRY(a_lp.ensure(m * gemm_ld(w->w.k) * 2));
        if (w->w.dtype >= COEUS_W_Q8_0) {
            int rc = w_lp.ensure(w->w.n * gemm_ld(w->w.k) * 2);
            if (rc != COEUS_OK) { a_lp.release(); return rc; }
        }
        scr.a_lp = a_lp.p; scr.a_lp_bytes = a_lp.bytes;
        scr.w_lp = w_lp.p; scr.w_lp_bytes = w_lp.bytes;
    }
    if (const uint64_t pb = gemm_split_scratch_bytes(w->w, m))
        if (part.ensure(pb) != COEUS_OK) part.release();
    scr.partials = (float *)part.p; scr.partials_bytes = part.bytes;
    int rc = launch_gemm(w->w, a_dev, m, e, scr, st);  // untimed first run
    hipEvent_t t0 = nullptr, t1 = nullptr;
    (void)hipEventCreate(&t0);
    (void)hipEventCreate(&t1);
    if (rc == COEUS_OK) {
        scr.repeat = reps; scr.ev_begin = t0; scr.ev_end = t1;
        rc = launch_gemm(w->w, a_dev, m, e, scr, st);
    }
    hipError_t se = hipStreamSynchronize(st);
    float ms = 0.f;
    if (rc == COEUS_OK && se == hipSuccess) se = hipEventElapsedTime(&ms, t0, t1);
    (void)hipEventDestroy(t0);
    (void)hipEventDestroy(t1);
    a_lp.release();
    w_lp.release();
    part.release();
    if (rc == COEUS_OK && se != hipSuccess) rc = fail(COEUS_DEVICE_ERROR, "matmul failed: %s", hipGetErrorString(se));
    *ms_out = ms;
    return rc;
    COEUS_GUARD_END
}

int coeus_op_norm(uint32_t kind, uint32_t scope, const float *x_dev, uint64_t rows, uint64_t hidden,
                  const float *scale_dev, const float *bias_dev, float eps, float *y_dev, void *stream) {
    COEUS_GUARD_BEGIN
    if (!x_dev || !scale_dev || !y_dev || (kind == COEUS_NORM_LAYERNORM && !bias_dev))
        return fail(COEUS_INVALID_INPUT, "null pointer argument");
    // whole-slice statistics over a large slice: many workgroups, through a scratch buffer that
    // lives for this call (the model keeps one in its workspace instead)
    double *part = nullptr;
    if (scope == COEUS_SCOPE_SEQUENCE && rows * hidden >= 32768)
        COEUS_HIP(hipMalloc((void **)&part, norm_sequence_scratch_bytes()));
    const int rc = launch_norm(kind, scope, x_dev, rows, hidden, scale_dev, bias_dev, eps, y_dev, nullptr, 0,
                               (hipStream_t)stream, nullptr, part);
    if (part) {
        (void)hipStreamSynchronize((hipStream_t)stream);
        (void)hipFree(part);
    }
    return rc;
    COEUS_GUARD_END
}

int coeus_op_embed(const float *table_dev, const float *pe_dev, const uint64_t *ids_dev, uint64_t rows,
                   uint64_t pos0, uint64_t hidden, float *x_dev, void *stream) {
    COEUS_GUARD_BEGIN
    if (!table_dev || !pe_dev || !ids_dev || !x_dev) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    return launch_embed(table_dev, false, pe_dev, ids_dev, rows, rows, pos0, nullptr, hidden, x_dev,
                        nullptr, (hipStream_t)stream);
    COEUS_GUARD_END
}

int coeus_op_attention(const float *qkv_dev, uint64_t rows, uint64_t num_heads, uint64_t head_dim,
                       float *out_dev, void *stream) {
    COEUS_GUARD_BEGIN
    if (!qkv_dev || !out_dev) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    if (rows == 0 || num_heads == 0) return fail(COEUS_INVALID_INPUT, "empty attention input");
    hipStream_t st = (hipStream_t)stream;
    DeviceBuf k, v;
    const uint64_t bytes = num_heads * rows * head_dim * 4;
    COEUS_TRY(k.ensure(bytes));
    int rc = v.ensure(bytes);
    if (rc == COEUS_OK)
        rc = launch_kv_append(qkv_dev, k.p, v.p, COEUS_KV_F32, 1, rows, num_heads, head_dim, rows, 0, nullptr, st);
    if (rc == COEUS_OK)
        rc = launch_attention(qkv_dev, k.p, v.p, COEUS_KV_F32, 1, rows, num_heads, head_dim, rows, 0,
                              nullptr, out_dev, nullptr, 0, nullptr, 0, nullptr, st);
    hipError_t se = hipStreamSynchronize(st);
    k.release();
    v.release();
    if (rc == COEUS_OK && se != hipSuccess) rc = fail(COEUS_DEVICE_ERROR, "attention failed: %s", hipGetErrorString(se));
    return rc;
    COEUS_GUARD_END
}

static int check_attention_decode_args(const float *qkv_dev, const void *k, const void *v, uint32_t kv_dtype,
                                       uint64_t batch, uint64_t heads, uint64_t hd, uint64_t max_ctx,
                                       uint64_t ctx, uint32_t *nsplit, uint32_t merge, const float *out_dev) {
    if (!qkv_dev || !k || !v || !out_dev) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    if (batch == 0 || heads == 0 || batch > 65535 || heads > 65535)
        return fail(COEUS_INVALID_INPUT, "decode attention: batch %llu x heads %llu out of range",
                    (unsigned long long)batch, (unsigned long long)heads);
    if (hd != 64 && hd != 128)
        return fail(COEUS_INVALID_INPUT, "decode attention: head_dim %llu is not 64 or 128", (unsigned long long)hd);
    if (kv_dtype != COEUS_KV_F16 && kv_dtype != COEUS_KV_BF16)
        return fail(COEUS_INVALID_INPUT, "decode attention: the cache must be f16 or bf16");
    // (the kernel indexes positions with 32 bits, like validate_config's bound on max_seq_len)
    if (max_ctx >= (1ull << 31))
        return fail(COEUS_INVALID_INPUT, "decode attention: max_ctx %llu out of range [1, 2^31)",
                    (unsigned long long)max_ctx);
    if (ctx == 0 || ctx > max_ctx)
        return fail(COEUS_INVALID_INPUT, "Sequence length %llu out of range [1, %llu]", (unsigned long long)ctx,
                    (unsigned long long)max_ctx);
    if (merge > COEUS_MERGE_SEPARATE) return fail(COEUS_INVALID_INPUT, "unknown merge mode %u", merge);
    if (*nsplit == 0) *nsplit = attn_decode_splits(batch, heads, max_ctx);
    if (*nsplit > 32) return fail(COEUS_INVALID_INPUT, "decode attention: %u splits out of range [1, 32]", *nsplit);
    return COEUS_OK;
}

int coeus_op_attention_decode(const float *qkv_dev, const void *k_cache_dev, const void *v_cache_dev,
                              uint32_t kv_dtype, uint64_t batch, uint64_t num_heads, uint64_t head_dim,
                              uint64_t max_ctx, uint64_t ctx, uint32_t nsplit, uint32_t merge,
                              float *out_dev, void *stream) {
    COEUS_GUARD_BEGIN
    COEUS_TRY(check_attention_decode_args(qkv_dev, k_cache_dev, v_cache_dev, kv_dtype, batch, num_heads, head_dim,
                                          max_ctx, ctx, &nsplit, merge, out_dev));
    hipStream_t st = (hipStream_t)stream;
    DeviceBuf part, count;
    COEUS_TRY(part.ensure(batch * num_heads * nsplit * (head_dim + 2) * 4));
    int rc = count.ensure(batch * num_heads * 4);
    hipError_t se = hipSuccess;
    if (rc == COEUS_OK) se = hipMemsetAsync(count.p, 0, count.bytes, st);
    if (rc == COEUS_OK && se == hipSuccess)
        rc = launch_attention(qkv_dev, k_cache_dev, v_cache_dev, kv_dtype, batch, 1, num_heads, head_dim, max_ctx,
                              ctx - 1, nullptr, out_dev, nullptr, 0, (float *)part.p, nsplit,
                              merge == COEUS_MERGE_IN_KERNEL ? (uint32_t *)count.p : nullptr, st);
    const hipError_t se2 = hipStreamSynchronize(st);
    part.release();
    count.release();
    if (rc == COEUS_OK && (se != hipSuccess || se2 != hipSuccess))
        rc = fail(COEUS_DEVICE_ERROR, "decode attention failed: %s", hipGetErrorString(se != hipSuccess ? se : se2));
    return rc;
    COEUS_GUARD_END
}

// ---------------------------------------------------------------- decode attention without allocation
// Device memory for coeus_op_attention_decode_static: the partial (max, sum, output) records of the
// context splits and the arrival counters of the in-kernel merge, in a file-scope array instead of
// a per-call allocation.  Every GPU the library runs on holds its own copy (2.04 MiB) until the
// process ends.  The array's name is only a host-side handle: device code is given the address
// that hipGetSymbolAddress returns for the current device.
constexpr uint64_t kStaticRecords = 4096;  // (sequence, head, split) triples of one call
constexpr uint64_t kStaticPairs = 1024;    // (sequence, head) pairs of one call
constexpr uint64_t kStaticRecordBytes = kStaticRecords * (128 + 2) * sizeof(float);
constexpr uint64_t kStaticScratchBytes = kStaticRecordBytes + kStaticPairs * sizeof(uint32_t);
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mu;
static void *g_scratch_ptr[kMaxDevices];  // per device: the address of its copy of `scratch`

static int static_scratch_for_current_device(unsigned char **out) {
    int dev = 0;
    COEUS_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(COEUS_DEVICE_ERROR, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        COEUS_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return fail(COEUS_DEVICE_ERROR, "hipGetSymbolAddress returned a null address");
        g_scratch_ptr[dev] = p;
    }
    *out = (unsigned char *)g_scratch_ptr[dev];
    return COEUS_OK;
}

__global__ void clear_u32_kernel(uint32_t *p, uint32_t n) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

int coeus_op_attention_decode_static(const float *qkv_dev, const void *k_cache_dev, const void *v_cache_dev,
                                     uint32_t kv_dtype, uint64_t batch, uint64_t num_heads, uint64_t head_dim,
                                     uint64_t max_ctx, uint64_t ctx, uint32_t nsplit, uint32_t merge,
                                     float *out_dev, void *stream) {
    COEUS_GUARD_BEGIN
    COEUS_TRY(check_attention_decode_args(qkv_dev, k_cache_dev, v_cache_dev, kv_dtype, batch, num_heads, head_dim,
                                          max_ctx, ctx, &nsplit, merge, out_dev));
    const uint64_t pairs = batch * num_heads, records = pairs * nsplit;
    if (pairs > kStaticPairs || records > kStaticRecords)
        return fail(COEUS_INVALID_INPUT,
                    "decode attention without allocation: batch %llu x heads %llu x splits %u needs %llu partial "
                    "records and %llu counters, the static buffer holds %llu and %llu",
                    (unsigned long long)batch, (unsigned long long)num_heads, nsplit, (unsigned long long)records,
                    (unsigned long long)pairs, (unsigned long long)kStaticRecords, (unsigned long long)kStaticPairs);
    unsigned char *base = nullptr;
    COEUS_TRY(static_scratch_for_current_device(&base));
    float *part = (float *)base;
    uint32_t *counters = (uint32_t *)(base + kStaticRecordBytes);
    hipStream_t st = (hipStream_t)stream;
    if (merge == COEUS_MERGE_IN_KERNEL) {
        // The merging split leaves its counter at zero, but a launch that was cut short would not:
        // clear them with a kernel (a memset node in a captured graph is not reliable here).
        hipLaunchKernelGGL(clear_u32_kernel, dim3((unsigned)ceil_div(pairs, 256)), dim3(256), 0, st, counters,
                           (uint32_t)pairs);
        COEUS_HIP(hipGetLastError());
    }
    return launch_attention(qkv_dev, k_cache_dev, v_cache_dev, kv_dtype, batch, 1, num_heads, head_dim, max_ctx,
                            ctx - 1, nullptr, out_dev, nullptr, 0, part, nsplit,
                            merge == COEUS_MERGE_IN_KERNEL ? counters : nullptr, st);
    COEUS_GUARD_END
}

}  // extern "C"
