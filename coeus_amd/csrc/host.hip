// Host-only part of libcoeus_mi355x.so: errors, Transformer250MConfig (default, validate),
// the parameter layout, the sinusoidal table, and the extern "C" entry points that never touch
// the device (configuration, .rustllm files, the reference's initialisation loop).  Together with
// rustllm_file.hip and bpe.hip this file builds without any device code, which is what the
// address / undefined-behaviour sanitizer build of the host logic links.
#include "model.hpp"

#include <cmath>
#include <new>

namespace coeus {

// ---------------------------------------------------------------- errors
static thread_local std::string g_error;

void set_error(const char *fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_error = buf;
}

int fail(int status, const char *fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_error = buf;
    return status;
}

const char *last_error() { return g_error.c_str(); }

// ---------------------------------------------------------------- profiler detection
// A rocprofiler-sdk tool in the process (rocprofv3 preloads librocprofiler-sdk-tool.so and names it
// in ROCP_TOOL_LIBRARIES) changes how captured graphs are replayed: a replay of a graph that holds
// the decode attention kernel has ended such a process with a host-side segmentation fault.
// Sessions therefore launch kernel by kernel whenever this returns true.  The answer is looked up
// once: from the environment that a tool's launcher sets and from the shared objects mapped into
// the process (read as text from /proc/self/maps; nothing is loaded or called).
static bool names_profiler_tool(const char *s) {
    return s && (strstr(s, "rocprofiler-sdk-tool") || strstr(s, "librocprofv") || strstr(s, "rocprof-sys") ||
                 strstr(s, "librocprofiler64") || strstr(s, "libroctracer64"));
}

bool profiler_attached() {
    static const bool attached = [] {
        const char *tool = getenv("ROCP_TOOL_LIBRARIES");
        if (tool && *tool) return true;
        for (const char *name : {"LD_PRELOAD", "HSA_TOOLS_LIB", "ROCPROFILER_LIBRARY_CTOR"})
            if (names_profiler_tool(getenv(name)) || (strcmp(name, "ROCPROFILER_LIBRARY_CTOR") == 0 && getenv(name)))
                return true;
        bool found = false;
        if (FILE *f = fopen("/proc/self/maps", "r")) {
            char line[1024];
            while (!found && fgets(line, sizeof(line), f)) found = names_profiler_tool(line);
            fclose(f);
        }
        return found;
    }();
    return attached;
}

// Why captured graphs must not be replayed in this process, or nullptr when they may: a profiler
// tool is attached, or the user asked for plain launches with COEUS_NO_GRAPH=1.
const char *graph_replay_forbidden() {
    if (profiler_attached())
        return "a rocprofiler tool library is loaded in this process: decode steps are launched kernel by "
               "kernel (replaying a captured decode step under the profiler has crashed the process)";
    const char *force = getenv("COEUS_NO_GRAPH");
    if (force && *force && strcmp(force, "0") != 0) return "COEUS_NO_GRAPH is set";
    return nullptr;
}

// ---------------------------------------------------------------- config + layout
// Transformer250MConfig::validate (CM:487-531), same order; extension fields afterwards.
int validate_config(const coeus_config &c) {
    auto bad = [](const char *key, unsigned long long value, const char *why) {
        return fail(COEUS_INVALID_CONFIG, "Invalid configuration: %s = %llu: %s", key, value, why);
    };
    if (c.hidden_dim == 0) return bad("hidden_dim", 0, "Hidden dimension must be greater than 0");
    if (c.num_heads == 0) return bad("num_heads", 0, "Number of heads must be greater than 0");
    if (c.head_dim == 0 && c.hidden_dim % c.num_heads != 0)
        return fail(COEUS_INVALID_CONFIG,
                    "Invalid configuration: hidden_dim = %llu (num_heads=%llu): Hidden dimension "
                    "must be divisible by number of heads",
                    (unsigned long long)c.hidden_dim, (unsigned long long)c.num_heads);
    if (c.num_layers == 0) return bad("num_layers", 0, "Number of layers must be greater than 0");
    if (c.vocab_size == 0) return bad("vocab_size", 0, "Vocabulary size must be greater than 0");
    if (c.max_seq_len == 0) return bad("max_seq_len", 0, "Maximum sequence length must be greater than 0");
    if (c.activation > COEUS_ACT_SILU_GATED) return bad("activation", c.activation, "unknown activation");
    if (c.norm > COEUS_NORM_RMSNORM) return bad("norm", c.norm, "unknown norm");
    if (c.norm_scope > COEUS_SCOPE_TOKEN) return bad("norm_scope", c.norm_scope, "unknown norm scope");
    if (c.weight_dtype > COEUS_W_Q4_0) return bad("weight_dtype", c.weight_dtype, "unknown weight dtype");
    if (c.kv_dtype > COEUS_KV_BF16) return bad("kv_dtype", c.kv_dtype, "unknown kv dtype");
    if (c.intermediate_dim == 0) return bad("intermediate_dim", 0, "Intermediate dimension must be greater than 0");
    const uint64_t hd = c.head_dim ? c.head_dim : c.hidden_dim / c.num_heads;
    if (hd > 256) return bad("head_dim", hd, "head dimension above 256 is not supported");
    if (c.max_batch > 16) return bad("max_batch", c.max_batch, "at most 16 sequences per session");
    if (c.max_seq_len >= (1ull << 31)) return bad("max_seq_len", c.max_seq_len, "too large");
    if (c.weight_dtype >= COEUS_W_Q8_0) {
        const uint64_t inner = c.num_heads * hd;
        if (c.hidden_dim % 32 || c.intermediate_dim % 32 || inner % 32)
            return fail(COEUS_INVALID_CONFIG,
                        "Invalid configuration: weight_dtype = %u: block-quantised weights need "
                        "hidden, intermediate and heads*head_dim divisible by 32",
                        c.weight_dtype);
    }
    return COEUS_OK;
}

Layout make_layout(const coeus_config &c) {
    Layout L{};
    const uint64_t H = c.hidden_dim, I = c.intermediate_dim, V = c.vocab_size;
    L.head_dim = c.head_dim ? c.head_dim : (c.num_heads ? H / c.num_heads : 0);
    const uint64_t inner = c.num_heads * L.head_dim;
    const bool gated = c.activation == COEUS_ACT_SILU_GATED;
    L.inner_dim = inner;
    L.token_embed_offset = 0;
    L.token_embed_size = V * H;          // MT:685-687
    L.first_layer_offset = V * H;
    uint64_t o = 0;                      // MT:695-721 / MT:839-880
    L.ln1_scale = o; o += H;
    L.ln1_bias = o;  o += H;
    L.wq = o; o += H * inner;
    L.wk = o; o += H * inner;
    L.wv = o; o += H * inner;
    L.wo = o; o += inner * H;
    if (c.use_bias) {
        L.bq = o; o += inner;
        L.bk = o; o += inner;
        L.bv = o; o += inner;
        L.bo = o; o += H;
    }
    L.ln2_scale = o; o += H;
    L.ln2_bias = o;  o += H;
    if (gated) { L.w_gate = o; o += H * I; }
    L.w_up = o;   o += H * I;
    L.w_down = o; o += I * H;
    if (c.use_bias) {
        if (gated) { L.b_gate = o; o += I; }
        L.b_up = o;   o += I;
        L.b_down = o; o += H;
    }
    L.layer_stride = o;
    L.final_ln_offset = L.first_layer_offset + c.num_layers * L.layer_stride;  // MT:724-726
    L.output_proj_offset = L.final_ln_offset + 2 * H;                          // MT:729-730
    L.output_proj_size = H * V;
    L.used_params = L.output_proj_offset + L.output_proj_size;
    // MT:546 and MT:575-577: counted by build(), never read by forward
    L.total_params = L.used_params + c.max_seq_len * H + (c.use_bias ? V : 0);
    return L;
}

// PositionalEncoding::new (MT:398-407), host libm like the reference.
void positional_encoding_host(uint64_t max_seq_len, uint64_t hidden, float *t) {
    std::memset(t, 0, sizeof(float) * max_seq_len * hidden);
    for (uint64_t pos = 0; pos < max_seq_len; pos++)
        for (uint64_t i = 0; i < hidden / 2; i++) {
            volatile float e = 2.0f * (float)i / (float)hidden;
            volatile float den = powf(10000.0f, e);
            const float angle = (float)pos / den;
            t[pos * hidden + 2 * i] = sinf(angle);
            t[pos * hidden + 2 * i + 1] = cosf(angle);
        }
}

}  // namespace coeus

using namespace coeus;

extern "C" {

const char *coeus_last_error(void) { return last_error(); }

int coeus_profiler_attached(void) { return profiler_attached() ? 1 : 0; }

void coeus_config_default(coeus_config *c) {
    if (!c) return;
    std::memset(c, 0, sizeof(*c));
    c->hidden_dim = 768;          // CM:537
    c->num_layers = 12;           // CM:538
    c->num_heads = 12;            // CM:539
    c->intermediate_dim = 3072;   // CM:540
    c->vocab_size = 50257;        // CM:541
    c->max_seq_len = 1024;        // CM:542
    c->dropout = 0.1f;            // CM:543
    c->attention_dropout = 0.1f;  // CM:544
    c->layer_norm_eps = 1e-5f;    // CM:545
    c->use_bias = 1;              // CM:546
}

int coeus_config_validate(const coeus_config *c) {
    if (!c) return fail(COEUS_INVALID_INPUT, "null config");
    return validate_config(*c);
}

uint64_t coeus_config_num_parameters(const coeus_config *c) { return c ? make_layout(*c).total_params : 0; }
uint64_t coeus_config_used_parameters(const coeus_config *c) { return c ? make_layout(*c).used_params : 0; }

uint64_t coeus_rustllm_checksum(const float *params, uint64_t n) {
    return params || n == 0 ? rustllm_checksum(params, n) : 0;
}
int coeus_rustllm_write(const char *path, const coeus_config *cfg, const float *params, uint64_t n) {
    COEUS_GUARD_BEGIN
    if (!path || !cfg || (!params && n)) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    return rustllm_write(path, *cfg, params, n);
    COEUS_GUARD_END
}
int coeus_rustllm_read_header(const char *path, coeus_config *cfg_out, uint64_t *n_params_out) {
    COEUS_GUARD_BEGIN
    if (!path || !cfg_out || !n_params_out) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    return rustllm_read_header(path, *cfg_out, *n_params_out);
    COEUS_GUARD_END
}
int coeus_rustllm_read_parameters(const char *path, float *params_out, uint64_t n) {
    COEUS_GUARD_BEGIN
    if (!path || (!params_out && n)) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    return rustllm_read_parameters(path, params_out, n);
    COEUS_GUARD_END
}

int coeus_init_default_parameters(float *params, uint64_t n, uint64_t hidden_dim) {
    if (!params && n) return fail(COEUS_INVALID_INPUT, "null parameter buffer");
    // MT:604-611; the index is converted to f32 before the multiply, as `i as f32` does
    const float hidden = (float)hidden_dim;
    const float scale = sqrtf(2.0f / hidden);
    for (uint64_t i = 0; i < n; i++) {
        volatile float arg = (float)i * 0.1234567f;
        float v = sinf(arg) * scale;
        if (v < -0.1f) v = -0.1f;
        if (v > 0.1f) v = 0.1f;
        params[i] = v;
    }
    return COEUS_OK;
}

int coeus_positional_encoding(uint64_t max_seq_len, uint64_t hidden_dim, float *table_out) {
    if (!table_out) return fail(COEUS_INVALID_INPUT, "null table");
    positional_encoding_host(max_seq_len, hidden_dim, table_out);
    return COEUS_OK;
}

}  // extern "C"
