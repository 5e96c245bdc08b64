// Model / session objects behind the C ABI.
#pragma once

#include <memory>

#include "common.hpp"

namespace coeus {

const char *last_error();
int validate_config(const coeus_config &c);
void positional_encoding_host(uint64_t max_seq_len, uint64_t hidden, float *table);
bool profiler_attached();
const char *graph_replay_forbidden();

struct DeviceBuf {
    void *p = nullptr;
    uint64_t bytes = 0;
    int ensure(uint64_t want);  // grows (contents are not preserved)
    void release();
};

struct LayerWeights {
    Weight qkv, o, up, down;  // up holds interleaved (gate, up) rows for a gated FFN
    const float *ln1_s = nullptr, *ln1_b = nullptr, *ln2_s = nullptr, *ln2_b = nullptr;
    const float *b_qkv = nullptr, *b_o = nullptr, *b_up = nullptr, *b_down = nullptr;
};

struct Model;

// Activation buffers of the matrix-core (prefill) path, grown on demand.
struct Workspace {
    uint64_t rows = 0;
    DeviceBuf h, x, qkv, att, ff, ids, a_lp, b_lp, w_lp, logits, xq, norm_part, gemm_part;
    GemmScratch gs;
    int ensure(const Model &m, uint64_t rows_needed, uint64_t logit_rows);
    void release();
};

struct Cache {
    void *k, *v;
    uint64_t max_ctx;
    uint64_t layer_bytes;
    bool per_layer;  // false: one layer's worth of storage reused by every layer
};

struct Model {
    coeus_config cfg{};
    Layout L{};
    uint64_t n_params = 0, weight_bytes = 0;
    std::vector<LayerWeights> layers;
    Weight out;
    void *embed = nullptr;
    bool embed_bf16 = false;
    float *pe = nullptr, *small = nullptr;
    const float *fin_s = nullptr, *fin_b = nullptr;
    hipStream_t stream = nullptr;
    std::mutex mu;  // serialises every call that touches the stream or the workspaces
    Workspace ws;
    DeviceBuf tmp_k, tmp_v;
    // HBM that resident f16 copies of quantised weights may still take (prefill matmul operands)
    static constexpr uint64_t kExpandBudget = 64ull << 30;
    uint64_t expand_budget = kExpandBudget;
    ~Model();
};

struct Session {
    Model *m = nullptr;
    uint64_t batch = 0, max_ctx = 0, pos = 0, layer_bytes = 0;
    uint32_t bp = 1, nsplit = 1;
    bool use_graph = true;
    bool fuse = true;  // fold norms into the decode matmuls where possible
    uint32_t host_pos[2] = {0, 0};
    DeviceBuf kc, vc;
    Workspace ws;  // prefill
    DeviceBuf dh, dx, dqkv, datt, dff, dlogits, dids, dpos, dhist, dpart, dcount, dstats, xq_h, xq_inner, xq_ff, xq_g;
    hipGraph_t graph = nullptr;
    hipGraphExec_t graph_exec = nullptr;
    ~Session();
};

int model_create(const coeus_config &cfg, const float *params, uint64_t n_params, uint64_t seed,
                 Model **out);
int model_forward(Model &m, const uint64_t *ids, uint64_t seq_len, float *logits_out, bool all_rows);
int session_create(Model &m, uint64_t batch, uint64_t max_ctx, Session **out);
int session_prefill(Session &s, const uint64_t *ids, uint64_t n, float *logits_out);
int session_decode(Session &s, const uint64_t *ids, float *logits_out);
int session_decode_greedy(Session &s, const uint64_t *first_ids, uint64_t n_steps, uint64_t *out_ids,
                          const coeus_sampling *sampling = nullptr);

int session_time_decode_matmuls(Session &s, uint64_t reps, float *ms_out, uint64_t *launches_out,
                                uint64_t *bytes_out);
int session_time_decode_attention(Session &s, uint64_t reps, float *ms_out, uint64_t *launches_out,
                                  uint64_t *bytes_out);

}  // namespace coeus
