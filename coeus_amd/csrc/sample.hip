// Token sampling from a row of logits (temperature, top-k, top-p): the step after the logits that
// the reference names but does not implement (BasicGenerationConfig, core/model.rs:718-753;
// GenerativeModel::generate, core/model.rs:138-144).
//
//   temperature <= 0  -> argmax (lowest index on ties)
//   candidates        -> the top_k (<= 64) largest logits in (value descending, index ascending)
//                        order, or the whole vocabulary in index order when top_k = 0
//   weight            -> floor(exp((z - z_max) / temperature) * 2^24), with an exponential built
//                        from f32 multiplies and adds only (this file is compiled without
//                        floating-point contraction), so a CPU restatement gets the same integers
//   top_p (with top_k)-> shortest candidate prefix whose weight reaches
//                        floor(top_p * 2^24) * total >> 24
//   draw              -> u24 = top 24 bits of splitmix64(seed ^ f(position, row)); the first
//                        candidate whose running weight sum exceeds (u24 * total) >> 24
// After the weights everything is integer arithmetic: the parallel sums below give exactly the
// result of a sequential loop.
#include "device_utils.hpp"

namespace coeus {

__device__ __forceinline__ uint64_t sample_mix(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

// exp(x) for x <= 0: Cody-Waite reduction, degree-7 Taylor polynomial in Horner form, exact scaling
__device__ __forceinline__ float exp_nonpositive(float x) {
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

__device__ __forceinline__ uint64_t sample_weight(float z, float zmax, float temperature) {
    return (uint64_t)(exp_nonpositive((z - zmax) / temperature) * 16777216.0f);
}

// (value, index) order: a comes before b
__device__ __forceinline__ bool before(float va, uint32_t ia, float vb, uint32_t ib) {
    return va > vb || (va == vb && ia < ib);
}

// Greatest element (in that order) over the block; every thread gets the result.
__device__ __forceinline__ void block_best(float &v, uint32_t &i, float *sv, uint32_t *si) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(v, off, 64);
        const uint32_t oi = __shfl_xor(i, off, 64);
        if (oi != 0xffffffffu && (i == 0xffffffffu || before(ov, oi, v, i))) { v = ov; i = oi; }
    }
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    __syncthreads();
    if (lane == 0) { sv[wave] = v; si[wave] = i; }
    __syncthreads();
    v = sv[0]; i = si[0];
    for (uint32_t w = 1; w < nw; w++)
        if (si[w] != 0xffffffffu && (i == 0xffffffffu || before(sv[w], si[w], v, i))) { v = sv[w]; i = si[w]; }
}

__device__ __forceinline__ uint64_t block_sum_u64(uint64_t v, uint64_t *sh) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    __syncthreads();
    if (lane == 0) sh[wave] = v;
    __syncthreads();
    uint64_t t = 0;
    for (uint32_t w = 0; w < nw; w++) t += sh[w];
    return t;
}

// One workgroup of 1024 threads per row.
__global__ __launch_bounds__(1024) void sample_kernel(const float *__restrict__ logits, uint32_t vocab,
                                                      uint32_t top_k, uint32_t top_p_fixed,
                                                      float temperature, uint64_t seed, uint64_t pos0,
                                                      const uint32_t *pos_dev, uint64_t *out_ids,
                                                      uint64_t *history, uint64_t history_stride,
                                                      const uint32_t *step_dev) {
    __shared__ float sv[16];
    __shared__ uint32_t si[16];
    __shared__ uint64_t s64[16];
    __shared__ float cand_v[64];
    __shared__ uint32_t cand_i[64];
    __shared__ uint64_t chunk_sum[1024];
    __shared__ uint32_t result;
    const uint32_t row = blockIdx.x, tid = threadIdx.x;
    const float *z = logits + (uint64_t)row * vocab;
    const uint64_t position = pos0 + (pos_dev ? (uint64_t)*pos_dev : 0);  // device part + host offset

    float bv = -INFINITY;
    uint32_t bi = 0xffffffffu;
    for (uint32_t i = tid; i < vocab; i += blockDim.x) {
        const float v = z[i];
        if (bi == 0xffffffffu ? v == v : before(v, i, bv, bi)) { bv = v; bi = i; }
    }
    block_best(bv, bi, sv, si);
    if (bi == 0xffffffffu) { bv = z[0]; bi = 0; }  // all NaN
    uint32_t pick = bi;
    const float zmax = bv;
    if (temperature > 0.0f && vocab > 1) {
        const uint64_t u24 = sample_mix(seed ^ ((position + 1) * 0xD1B54A32D192ED03ull) ^
                                        (((uint64_t)row + 1) * 0x9E3779B97F4A7C15ull)) >> 40;
        if (top_k == 0) {
            // thread t owns the contiguous indices [t * per, (t + 1) * per)
            const uint32_t per = (vocab + blockDim.x - 1) / blockDim.x;
            const uint32_t i0 = min(tid * per, vocab), i1 = min(i0 + per, vocab);
            uint64_t mine = 0;
            for (uint32_t i = i0; i < i1; i++) mine += sample_weight(z[i], zmax, temperature);
            chunk_sum[tid] = mine;
            const uint64_t total = block_sum_u64(mine, s64);  // (syncs: chunk_sum is visible after it)
            const uint64_t target = (u24 * total) >> 24;
            if (tid == 0) result = bi;
            __syncthreads();
            // every thread finds its exclusive prefix; the one whose range holds the target scans it
            uint64_t excl = 0;
            for (uint32_t t = 0; t < tid; t++) excl += chunk_sum[t];
            if (target >= excl && target < excl + mine) {
                uint64_t run = excl;
                for (uint32_t i = i0; i < i1; i++) {
                    run += sample_weight(z[i], zmax, temperature);
                    if (run > target) { result = i; break; }
                }
            }
            __syncthreads();
            pick = result;
        } else {
            const uint32_t k = min(min(top_k, 64u), vocab);
            uint32_t found = 0;
            float pv = 0.f;
            uint32_t pi = 0;
            for (uint32_t j = 0; j < k; j++) {
                float cv = -INFINITY;
                uint32_t ci = 0xffffffffu;
                for (uint32_t i = tid; i < vocab; i += blockDim.x) {
                    const float v = z[i];
                    if (j > 0 && !(v < pv || (v == pv && i > pi))) continue;
                    if (ci == 0xffffffffu ? v == v : before(v, i, cv, ci)) { cv = v; ci = i; }
                }
                block_best(cv, ci, sv, si);
                if (ci == 0xffffffffu) break;  // uniform
                if (tid == 0) { cand_v[j] = cv; cand_i[j] = ci; }
                pv = cv; pi = ci;
                found = j + 1;
            }
            __syncthreads();
            if (tid == 0) result = bi;  // no candidate at all (a row of NaN): the argmax fallback
            __syncthreads();
            if (found > 0 && tid < 64) {  // wave 0: lane j owns candidate j (found is uniform)
                const uint64_t w = tid < found ? sample_weight(cand_v[tid], zmax, temperature) : 0;
                uint64_t incl = w;  // inclusive prefix sum over the lanes
#pragma unroll
                for (int off = 1; off < 64; off <<= 1) {
                    const uint64_t o = __shfl_up(incl, off, 64);
                    if ((int)tid >= off) incl += o;
                }
                uint64_t total = __shfl(incl, 63, 64);
                uint32_t m = found;
                if (top_p_fixed > 0 && top_p_fixed < (1u << 24)) {
                    const uint64_t thr = ((uint64_t)top_p_fixed * total) >> 24;
                    // the first lane whose inclusive sum reaches the threshold closes the nucleus
                    const uint64_t reach = __ballot(tid < found && incl >= thr);
                    m = reach ? (uint32_t)__ffsll((long long)reach) : found;
                    total = __shfl(incl, (int)m - 1, 64);
                }
                const uint64_t target = (u24 * total) >> 24;
                const uint64_t hit = __ballot(tid < m && incl > target);
                const uint32_t j = hit ? (uint32_t)__ffsll((long long)hit) - 1 : 0;
                if (tid == 0) result = cand_i[j];
            }
            __syncthreads();
            pick = result;
        }
    }
    if (tid == 0) {
        out_ids[row] = pick;
        if (history) history[(uint64_t)row * history_stride + (step_dev ? *step_dev : 0)] = pick;
    }
}

int launch_sample(const float *logits, uint64_t rows, uint64_t vocab, const coeus_sampling &cfg,
                  uint64_t pos0, const uint32_t *pos_dev, uint64_t *out_ids, uint64_t *history,
                  uint64_t history_stride, const uint32_t *step_dev, hipStream_t st) {
    if (rows == 0 || vocab == 0 || vocab > 0xfffffffeull) return fail(COEUS_INVALID_INPUT, "bad sampling shape");
    if (cfg.top_k > 64) return fail(COEUS_INVALID_INPUT, "top_k %u out of range [0, 64]", cfg.top_k);
    if (cfg.top_p > 0.f && cfg.top_p < 1.f && cfg.top_k == 0)
        return fail(COEUS_INVALID_INPUT, "top_p needs top_k (the nucleus is cut from the top_k candidates)");
    const uint32_t top_p_fixed = (cfg.top_p > 0.f && cfg.top_p < 1.f) ? (uint32_t)(cfg.top_p * 16777216.0f) : 0;
    hipLaunchKernelGGL(sample_kernel, dim3((unsigned)rows), dim3(1024), 0, st, logits, (uint32_t)vocab,
                       cfg.top_k, top_p_fixed, cfg.temperature, cfg.seed, pos0, pos_dev, out_ids, history,
                       history_stride, step_dev);
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

}  // namespace coeus
