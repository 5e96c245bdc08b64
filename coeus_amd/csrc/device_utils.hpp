// Device-side helpers shared by the kernels (gfx950, wave64).
#pragma once

#include "common.hpp"

namespace coeus {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

// Streaming (non-temporal) 16-byte load: data that is read exactly once should not displace
// the activations and scales that every workgroup re-reads from the caches.
__device__ __forceinline__ uint4 load_stream(const uint4 *p) {
    const u32x4_t v = __builtin_nontemporal_load((const u32x4_t *)p);
    return make_uint4(v.x, v.y, v.z, v.w);
}
typedef float float16_t __attribute__((ext_vector_type(16)));

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every
// outstanding global load of the wave (s_waitcnt vmcnt(0)), which drains a prefetch pipeline at
// each barrier; this one waits for LDS/scalar operations (lgkmcnt) and leaves loads in flight.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_s_waitcnt(0xC07F);  // vmcnt = 63 (no wait), expcnt = 7, lgkmcnt = 0
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Cross-lane reductions without LDS.  __shfl_xor compiles to ds_bpermute_b32, a round trip through
// the LDS pipe per step; the data-parallel-primitive modifiers (lane permutations within a row of
// 16 lanes, applied on the operand read of a VALU instruction) and the row / half swaps
// (v_permlane16_swap, v_permlane32_swap) are register moves.  Every lane of the wave must be
// active, and every lane receives the result.
template <int CTRL, int ROWS = 0xf>
__device__ __forceinline__ float dpp_f32(float v, float idle = 0.f) {  // lanes permuted by CTRL within their row
    // (a lane whose source lane is switched off, or whose row is not in ROWS, receives `idle`)
    return __uint_as_float(__builtin_amdgcn_update_dpp(__float_as_uint(idle), __float_as_uint(v), CTRL, ROWS, 0xf, false));
}
constexpr int DPP_QUAD_XOR1 = 0xB1, DPP_QUAD_XOR2 = 0x4E;  // quad_perm:[1,0,3,2], [2,3,0,1]
constexpr int DPP_ROW_ROR4 = 0x124, DPP_ROW_ROR8 = 0x128;  // rotate within the 16 lanes of a row
constexpr int DPP_HALF_MIRROR = 0x141;                     // reverse within 8 lanes
__device__ __forceinline__ float lane_xor1(float v) { return dpp_f32<DPP_QUAD_XOR1>(v); }
// Sum over the aligned group of N lanes (8 or 16) a lane belongs to.
template <int N>
__device__ __forceinline__ float group_sum(float v) {
    static_assert(N == 8 || N == 16, "group of 8 or 16 lanes");
    v += dpp_f32<DPP_QUAD_XOR1>(v);
    v += dpp_f32<DPP_QUAD_XOR2>(v);  // the quad's sum in its four lanes
    if (N == 8) {
        v += dpp_f32<DPP_HALF_MIRROR>(v);  // lane i of 8 meets lane 7 - i: the other quad
    } else {
        v += dpp_f32<DPP_ROW_ROR4>(v);  // this quad + the next
        v += dpp_f32<DPP_ROW_ROR8>(v);  // + the other two
    }
    return v;
}
// v of this lane + v of lane ^ 16 / lane ^ 32 (the swaps hand every lane both values)
__device__ __forceinline__ float xor16_sum(float v) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float xor32_sum(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
// The wave-wide sum stays on ds_bpermute: in the decode matmul's folded norm, where it matters, the
// LDS round trips overlap the weight unpacking, while a chain of six dependent DPP / swap
// instructions sits in the VALU stream (measured: 9.5 us per launch against 9.9 us).
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_f32<DPP_QUAD_XOR1>(v, v));
    v = fmaxf(v, dpp_f32<DPP_QUAD_XOR2>(v, v));
    v = fmaxf(v, dpp_f32<DPP_ROW_ROR4>(v, v));
    v = fmaxf(v, dpp_f32<DPP_ROW_ROR8>(v, v));
    auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float x) {
    uint32_t u = __float_as_uint(x);
    if ((u & 0x7f800000u) == 0x7f800000u && (u & 0x007fffffu)) return (uint16_t)((u | 0x00400000u) >> 16);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// math::gelu (MT:94-99)
__device__ __forceinline__ float gelu_tanh(float x) {
    const float c0 = 0.7978845608028654f, c1 = 0.044715f;
    return 0.5f * x * (1.0f + tanhf(c0 * x * (1.0f + c1 * x * x)));
}
__device__ __forceinline__ float silu(float x) { return x / (1.0f + expf(-x)); }
// The same activations on the hardware's exp2 and reciprocal (1 ulp each) for kernels whose
// epilogue is their tail: x * sigmoid(x), and 0.5 x (1 + tanh(u)) = x * sigmoid(2 u).
__device__ __forceinline__ float fast_sigmoid(float x) {
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x));
}
__device__ __forceinline__ float fast_silu(float x) { return x * fast_sigmoid(x); }
__device__ __forceinline__ float fast_gelu(float x) {
    const float c0 = 0.7978845608028654f, c1 = 0.044715f;
    return x * fast_sigmoid(2.0f * c0 * x * (1.0f + c1 * x * x));
}

// Position of element (b, k) in the xq interchange format ([k_pad/8][bp][8] f16).
__device__ __forceinline__ uint64_t xq_index(uint64_t k, uint32_t b, uint32_t bp) {
    return ((k >> 3) * bp + b) * 8 + (k & 7);
}

struct EpiArgs {
    const float *bias;
    const float *residual;
    float *out_f32;
    __half *out_xq;
    uint32_t act, bp_out;
    uint64_t n;      // weight rows (outputs before gating)
    uint64_t n_eff;  // outputs written per activation row (n, or n/2 when gated)
    // fused q|k|v projection of a decode step: columns >= kv_inner go straight into the cache
    void *kv_k, *kv_v;
    const uint32_t *kv_pos;
    uint32_t kv_dtype, kv_inner, kv_heads, kv_hd, kv_max_ctx;
    // prompt pass (kv_rows_per_seq > 0): row r is token r % kv_rows_per_seq of sequence
    // r / kv_rows_per_seq and goes to position kv_pos0 + r % kv_rows_per_seq
    uint32_t kv_rows_per_seq, kv_pos0;
    // per-(row, 16 outputs) statistics of the stored values, for the normalisation that the
    // consumer of these outputs folds into its staging: [rows][stats_tiles] {sum, M2}
    float2 *stats_out;
    uint32_t stats_tiles;
    // value * g_scale[j] for the consumer's root-mean-square norm (gemv_quad_kernel)
    const float *g_scale;
    float *g_out;
    // 16-bit copy of the output for the next prefill matmul (row stride lp_ld elements)
    uint16_t *out_lp;
    uint32_t lp_ld, lp_bf16;
};

__device__ __forceinline__ uint16_t f32_to_lp_bits(float v, bool bf16) {
    if (bf16) return f32_to_bf16_bits(v);
    union { _Float16 h; uint16_t u; } cv;
    cv.h = (_Float16)v;
    return cv.u;
}

// Statistics of 16 consecutive values of one activation row, held one per lane by the 16 lanes
// that share lane / 16: {sum, M2 = sum of squared deviations from the mean of these values}.
// `cnt` (1..16) values are real; lanes beyond pass live = false.  Every lane of the group must
// call this.  The consumer merges the records of a row: mean = sum(sum_t) / k and
// variance * k = sum(M2_t + cnt_t * (sum_t / cnt_t - mean)^2), or for a root-mean-square norm
// sum(x^2) = sum(M2_t + sum_t^2 / cnt_t).
// (register-to-register lane permutations: the matmul epilogues that call this are the tail of their
// kernels, and eight dependent trips through the LDS pipe were a third of that tail)
__device__ __forceinline__ float2 group16_stats(float v, bool live, uint32_t cnt) {
    const float s = group_sum<16>(live ? v : 0.f);
    const float d = live ? v - s * (cnt == 16 ? 0.0625f : 1.0f / (float)cnt) : 0.f;
    const float m2 = group_sum<16>(d * d);
    return make_float2(s, m2);
}

__device__ __forceinline__ void kv_cache_store(void *base, uint32_t kv_dtype, uint64_t idx, float v) {
    if (kv_dtype == COEUS_KV_F32) ((float *)base)[idx] = v;
    else if (kv_dtype == COEUS_KV_F16) ((__half *)base)[idx] = __float2half_rn(v);
    else ((uint16_t *)base)[idx] = f32_to_bf16_bits(v);
}

// Applies bias / activation / residual to one output element and stores it.
// `row` indexes the activation row (batch entry), `j` the output column.
// Returns the value stored.
// With `preloaded`, `res` is the residual element (row, j) fetched earlier by the caller.
// With `pos_known`, `pos` is *e.kv_pos read earlier by the caller.
template <bool KV = false>
__device__ __forceinline__ float epi_store(const EpiArgs &e, uint64_t row, uint64_t j, float v,
                                           bool preloaded = false, float res = 0.f, bool pos_known = false,
                                           uint32_t pos = 0) {
    if (e.bias) v += e.bias[j];
    if (KV && e.kv_k && j >= e.kv_inner) {
        // column j of q|k|v: key or value element (head, dim) of sequence `row` at position *kv_pos
        const uint32_t c = (uint32_t)(j % e.kv_inner), hh = c / e.kv_hd, d = c % e.kv_hd;
        const uint64_t idx = ((row * e.kv_heads + hh) * e.kv_max_ctx + (pos_known ? pos : *e.kv_pos)) * e.kv_hd + d;
        kv_cache_store(j < 2 * (uint64_t)e.kv_inner ? e.kv_k : e.kv_v, e.kv_dtype, idx, v);
        return v;
    }
    if (e.act == COEUS_EPI_GELU) v = gelu_tanh(v);
    if (e.residual) v += preloaded ? res : e.residual[row * e.n_eff + j];
    if (e.out_f32) e.out_f32[row * e.n_eff + j] = v;
    if (e.out_xq) e.out_xq[xq_index(j, (uint32_t)row, e.bp_out)] = __float2half_rn(v);
    if (e.out_lp) e.out_lp[row * e.lp_ld + j] = f32_to_lp_bits(v, e.lp_bf16);
    return v;
}
// Gated pair: rows (2m, 2m+1) of the weight hold gate_m and up_m; bias is interleaved alike.
__device__ __forceinline__ void epi_store_gated(const EpiArgs &e, uint64_t row, uint64_t m, float g,
                                                float u) {
    if (e.bias) { g += e.bias[2 * m]; u += e.bias[2 * m + 1]; }
    float v = silu(g) * u;
    if (e.residual) v += e.residual[row * e.n_eff + m];
    if (e.out_f32) e.out_f32[row * e.n_eff + m] = v;
    if (e.out_xq) e.out_xq[xq_index(m, (uint32_t)row, e.bp_out)] = __float2half_rn(v);
    if (e.out_lp) e.out_lp[row * e.lp_ld + m] = f32_to_lp_bits(v, e.lp_bf16);
}

static inline EpiArgs make_epi(const Epilogue &ep, uint64_t n) {
    EpiArgs e;
    e.bias = ep.bias;
    e.residual = ep.residual;
    e.out_f32 = ep.out_f32;
    e.out_xq = ep.out_xq;
    e.act = ep.act;
    e.bp_out = ep.bp_out;
    e.n = n;
    e.n_eff = ep.act == COEUS_EPI_SILU_GATE ? n / 2 : n;
    e.kv_k = ep.kv_k;
    e.kv_v = ep.kv_v;
    e.kv_pos = ep.kv_pos;
    e.kv_dtype = ep.kv_dtype;
    e.kv_inner = ep.kv_inner;
    e.kv_heads = ep.kv_heads;
    e.kv_hd = ep.kv_hd;
    e.kv_max_ctx = ep.kv_max_ctx;
    e.kv_rows_per_seq = ep.kv_rows_per_seq;
    e.kv_pos0 = ep.kv_pos0;
    e.stats_out = ep.stats_out;
    e.stats_tiles = (uint32_t)((e.n_eff + 15) / 16);
    e.g_scale = ep.g_scale;
    e.g_out = ep.g_out;
    e.out_lp = (uint16_t *)ep.out_lp.p;
    e.lp_ld = (uint32_t)ep.out_lp.ld;
    e.lp_bf16 = ep.out_lp.bf16 ? 1u : 0u;
    return e;
}

}  // namespace coeus
