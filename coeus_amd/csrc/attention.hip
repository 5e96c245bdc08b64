// Causal multi-head attention over an HBM-resident KV cache (MT:219-278: scores = q.k^T scaled
// AFTER the dot by 1/sqrt(head_dim), j > i masked, row softmax, P.V), evaluated with a running
// (online) softmax so no [seq, seq] score matrix or mask tensor is ever materialised.
//
// Cache layout: [batch][head][max_ctx][head_dim] per layer, element type f32 / f16 / bf16.
//
//   kv_append_kernel      scatters the k|v thirds of a projected qkv buffer into the cache.
//   attn_generic_kernel   one wave per (query row, head, sequence); lanes own keys for q.k and
//                         own output dimensions for P.V.  Any head_dim, any cache type.
//   attn_decode_kernel    one query per (sequence, head), head_dim 64 or 128, 16-bit cache: the
//                         context is split over workgroups (flash-decoding); every lane streams
//                         16-byte pieces of K and V with the same (key, dims) ownership in both
//                         phases, so probabilities never leave registers; a second kernel merges
//                         the per-split (max, sum, partial output) triples.
#include "device_utils.hpp"

namespace coeus {

template <typename T> __device__ __forceinline__ float kv_load(const T *p);
template <> __device__ __forceinline__ float kv_load<float>(const float *p) { return *p; }
template <> __device__ __forceinline__ float kv_load<__half>(const __half *p) { return __half2float(*p); }
template <> __device__ __forceinline__ float kv_load<uint16_t>(const uint16_t *p) { return bf16_bits_to_f32(*p); }

template <typename T> __device__ __forceinline__ T kv_store(float v);
template <> __device__ __forceinline__ float kv_store<float>(float v) { return v; }
template <> __device__ __forceinline__ __half kv_store<__half>(float v) { return __float2half_rn(v); }
template <> __device__ __forceinline__ uint16_t kv_store<uint16_t>(float v) { return f32_to_bf16_bits(v); }

// qkv [batch*n, 3*inner] f32 (q|k|v per row) -> cache rows pos0..pos0+n-1 of every sequence.
template <typename T>
__global__ void kv_append_kernel(const float *__restrict__ qkv, T *kc, T *vc, uint32_t n,
                                 uint32_t heads, uint32_t hd, uint32_t max_ctx, uint32_t pos0,
                                 const uint32_t *pos_dev) {
    const uint32_t inner = heads * hd;
    const uint64_t row = blockIdx.x;  // b*n + i
    const uint32_t b = (uint32_t)(row / n), i = (uint32_t)(row % n);
    const uint32_t pos = (pos_dev ? *pos_dev : pos0) + i;
    for (uint32_t c = threadIdx.x; c < inner; c += blockDim.x) {
        const uint32_t h = c / hd, d = c % hd;
        const uint64_t dst = (((uint64_t)b * heads + h) * max_ctx + pos) * hd + d;
        kc[dst] = kv_store<T>(qkv[row * 3 * inner + inner + c]);
        vc[dst] = kv_store<T>(qkv[row * 3 * inner + 2 * inner + c]);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void attn_generic_kernel(const float *__restrict__ qkv,
                                                           const T *__restrict__ kc,
                                                           const T *__restrict__ vc, uint32_t n,
                                                           uint32_t heads, uint32_t hd,
                                                           uint32_t max_ctx, uint32_t pos0,
                                                           const uint32_t *pos_dev, float *out,
                                                           __half *out_xq, uint32_t bp) {
    extern __shared__ float lds[];  // per wave: q[hd] + p[64]
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t i = blockIdx.x * 4 + wave, h = blockIdx.y, b = blockIdx.z;
    if (i >= n) return;
    const uint32_t inner = heads * hd;
    float *qs = lds + wave * (hd + 64), *ps = qs + hd;
    const uint64_t row = (uint64_t)b * n + i;
    for (uint32_t d = lane; d < hd; d += 64) qs[d] = qkv[row * 3 * inner + h * hd + d];
    const uint32_t ctx = (pos_dev ? *pos_dev : pos0) + i + 1;  // keys 0..pos+i (causal)
    const T *kb = kc + ((uint64_t)b * heads + h) * max_ctx * hd;
    const T *vb = vc + ((uint64_t)b * heads + h) * max_ctx * hd;
    const float scale = 1.0f / sqrtf((float)hd);
    float m = -INFINITY, l = 0.f, acc0 = 0.f, acc1 = 0.f, acc2 = 0.f, acc3 = 0.f;  // hd <= 256
    for (uint32_t j0 = 0; j0 < ctx; j0 += 64) {
        const uint32_t j = j0 + lane;
        float s = -INFINITY;
        if (j < ctx) {
            float dot = 0.f;
            const T *kr = kb + (uint64_t)j * hd;
            for (uint32_t d = 0; d < hd; d++) dot = fmaf(qs[d], kv_load<T>(kr + d), dot);
            s = dot * scale;
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float p = j < ctx ? expf(s - m_new) : 0.f;
        const float corr = expf(m - m_new);  // first tile: exp(-inf) = 0
        l = l * corr + wave_sum(p);
        m = m_new;
        ps[lane] = p;
        acc0 *= corr; acc1 *= corr; acc2 *= corr; acc3 *= corr;
        const uint32_t cnt = min(64u, ctx - j0);
        for (uint32_t jj = 0; jj < cnt; jj++) {
            const float pj = ps[jj];
            const T *vr = vb + (uint64_t)(j0 + jj) * hd;
            if (lane < hd) acc0 = fmaf(pj, kv_load<T>(vr + lane), acc0);
            if (lane + 64 < hd) acc1 = fmaf(pj, kv_load<T>(vr + lane + 64), acc1);
            if (lane + 128 < hd) acc2 = fmaf(pj, kv_load<T>(vr + lane + 128), acc2);
            if (lane + 192 < hd) acc3 = fmaf(pj, kv_load<T>(vr + lane + 192), acc3);
        }
    }
    const float inv = 1.0f / l;
    const float r[4] = {acc0 * inv, acc1 * inv, acc2 * inv, acc3 * inv};
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const uint32_t d = lane + 64 * t;
        if (d < hd) {
            if (out) out[row * inner + h * hd + d] = r[t];
            if (out_xq) out_xq[xq_index(h * hd + d, (uint32_t)row, bp)] = __float2half_rn(r[t]);
        }
    }
}

// ---------------------------------------------------------------- flash-decoding (n == 1)
constexpr uint32_t kAttnMaxSplits = 32;  // splits per (sequence, head): bounds the merge's LDS
// Lane l owns 16-byte piece (l % CPK) of key (l / CPK) of every wave-wide load, CPK = HD/8.
template <int HD, bool BF16, int NW = 4>
__global__ __launch_bounds__(NW * 64) void attn_decode_kernel(const float *__restrict__ qkv,
                                                          const uint16_t *__restrict__ kc,
                                                          const uint16_t *__restrict__ vc,
                                                          uint32_t heads, uint32_t max_ctx,
                                                          uint32_t pos0, const uint32_t *pos_dev,
                                                          uint32_t keys_per_split, float *part,
                                                          uint32_t *counters, float *out,
                                                          __half *out_xq, uint32_t bp) {
    constexpr int CPK = HD / 8, KPL = 64 / CPK;  // pieces per key, keys per wave load
    constexpr int TILE = 16;                     // wave loads kept in flight per phase
    __shared__ float sm[NW], sl[NW], sacc[NW][HD];
    __shared__ float srec[kAttnMaxSplits * (HD + 2)];  // the partial records, for the merging split
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t split = blockIdx.x, h = blockIdx.y, b = blockIdx.z, nsplit = gridDim.x;
    const uint32_t inner = heads * HD;
    const uint32_t ctx = (pos_dev ? *pos_dev : pos0) + 1;
    const uint32_t piece = lane % CPK, ksub = lane / CPK;
    float q[8];
#pragma unroll
    for (int t = 0; t < 8; t++) q[t] = qkv[(uint64_t)b * 3 * inner + h * HD + piece * 8 + t];
    const uint64_t base = ((uint64_t)b * heads + h) * max_ctx * HD;
    const uint4 *k4 = (const uint4 *)(kc + base), *v4 = (const uint4 *)(vc + base);
    const uint32_t k_begin = split * keys_per_split;
    const uint32_t k_end = min(ctx, k_begin + keys_per_split);
    // scores and running maxima are kept in base 2: s = (q . k) * scale * log2(e), p = 2^(s - m):
    // one hardware exponential per key instead of expf's range reduction (this wave's sixteen keys
    // are evaluated after its last line has arrived, on the launch's tail)
    const float scale = 1.4426950408889634f / sqrtf((float)HD);
    float m = -INFINITY, l = 0.f, acc[8];
#pragma unroll
    for (int t = 0; t < 8; t++) acc[t] = 0.f;

    // each wave takes tiles of TILE*KPL keys, interleaved over the NW waves
    for (uint32_t t0 = k_begin + wave * TILE * KPL; t0 < k_end; t0 += NW * TILE * KPL) {
        // keys and values are requested together: the values do not depend on the scores, and
        // asking for them only after the scores exposed the memory latency a second time
        // Every load is unconditional, keys past the end re-reading the last one (their scores
        // are masked below, so their probabilities are zero): with loads under a branch the
        // compiler waits for all 32 before the first dot product, without it the scores start
        // when the first keys arrive.  Keys and values are read once per step: non-temporal loads
        // stream them faster (7B shape, context 4096, per step: batch 1 1.762 -> 1.752 ms, batch 4
        // 4.12 -> 3.93, batch 16 7.6-7.9 -> 7.5, the batch-16 launch 177 -> 167 us; 1B shape batch
        // 4 1.27 -> 1.17 ms; 250M Q8_0 batch 8 0.604 -> 0.566 ms).
        uint4 kr[TILE], vr[TILE];
#pragma unroll
        for (int t = 0; t < TILE; t++) {
            const uint32_t key = min(t0 + t * KPL + ksub, k_end - 1);
            kr[t] = load_stream(k4 + (uint64_t)key * CPK + piece);
        }
#pragma unroll
        for (int t = 0; t < TILE; t++) {
            const uint32_t key = min(t0 + t * KPL + ksub, k_end - 1);
            vr[t] = load_stream(v4 + (uint64_t)key * CPK + piece);
        }
        __builtin_amdgcn_sched_barrier(0);  // all 32 requests go out before anything is computed
        float s[TILE], tmax = -INFINITY;
#pragma unroll
        for (int t = 0; t < TILE; t++) {
            const uint32_t w[4] = {kr[t].x, kr[t].y, kr[t].z, kr[t].w};
            float dot = 0.f;
#pragma unroll
            for (int u = 0; u < 4; u++) {
                float lo, hi;
                if (BF16) { lo = __uint_as_float(w[u] << 16); hi = __uint_as_float(w[u] & 0xffff0000u); }
                else { union { uint32_t u32; half2_t h2; } cv; cv.u32 = w[u]; lo = (float)cv.h2.x; hi = (float)cv.h2.y; }
                dot = fmaf(q[2 * u], lo, dot);
                dot = fmaf(q[2 * u + 1], hi, dot);
            }
            // sum the CPK pieces of a key (the lanes of one key are an aligned group of 8 or 16)
            dot = group_sum<CPK>(dot);
            const uint32_t key = t0 + t * KPL + ksub;
            s[t] = key < k_end ? dot * scale : -INFINITY;
            tmax = fmaxf(tmax, s[t]);
        }
        const float m_new = fmaxf(m, wave_max(tmax));
        const float corr = __builtin_amdgcn_exp2f(m - m_new);
        float psum = 0.f;
#pragma unroll
        for (int t = 0; t < 8; t++) acc[t] *= corr;
#pragma unroll
        for (int t = 0; t < TILE; t++) {
            const float p = __builtin_amdgcn_exp2f(s[t] - m_new);  // 2^(-inf) = 0 for keys past the end
            psum += p;
            const uint32_t w[4] = {vr[t].x, vr[t].y, vr[t].z, vr[t].w};
#pragma unroll
            for (int u = 0; u < 4; u++) {
                float lo, hi;
                if (BF16) { lo = __uint_as_float(w[u] << 16); hi = __uint_as_float(w[u] & 0xffff0000u); }
                else { union { uint32_t u32; half2_t h2; } cv; cv.u32 = w[u]; lo = (float)cv.h2.x; hi = (float)cv.h2.y; }
                acc[2 * u] = fmaf(p, lo, acc[2 * u]);
                acc[2 * u + 1] = fmaf(p, hi, acc[2 * u + 1]);
            }
        }
        // every lane of a key holds the same p: count each key once
        l = l * corr + wave_sum(psum) * (1.0f / CPK);
        m = m_new;
    }
    // fold the KPL key-subsets of the wave: lanes with equal piece hold partial sums
#pragma unroll
    for (int t = 0; t < 8; t++) {
        if (CPK == 8) acc[t] += dpp_f32<DPP_ROW_ROR8>(acc[t]);  // the other 8 lanes of the row
        acc[t] = xor32_sum(xor16_sum(acc[t]));
    }
    if (lane == 0) { sm[wave] = m; sl[wave] = l; }
    if (lane < CPK)
#pragma unroll
        for (int t = 0; t < 8; t++) sacc[wave][lane * 8 + t] = acc[t];
    __syncthreads();
    // merge the waves; thread d < HD finishes output dimension d
    if (threadIdx.x < HD) {
        float mm = sm[0];
#pragma unroll
        for (int w = 1; w < NW; w++) mm = fmaxf(mm, sm[w]);
        float lt = 0.f, a = 0.f;
#pragma unroll
        for (int w = 0; w < NW; w++) {
            const float c = sm[w] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(sm[w] - mm);
            lt += sl[w] * c;
            a += sacc[w][threadIdx.x] * c;
        }
        if (nsplit == 1) {
            // the whole context in one workgroup: this is the result, nothing to publish or merge
            const float r = a / lt;
            if (out) out[(uint64_t)b * inner + h * HD + threadIdx.x] = r;
            if (out_xq) out_xq[xq_index(h * HD + threadIdx.x, b, bp)] = __float2half_rn(r);
            return;
        }
        // partial record per (b, h, split): [m, l, acc[HD]]
        float *rec = part + (((uint64_t)b * heads + h) * nsplit + split) * (HD + 2);
        if (counters) {
            // device-scope stores: written through to the point where every XCD sees them
            if (threadIdx.x == 0) {
                __hip_atomic_store(rec, mm, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(rec + 1, lt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            __hip_atomic_store(rec + 2 + threadIdx.x, a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
            if (threadIdx.x == 0) { rec[0] = mm; rec[1] = lt; }
            rec[2 + threadIdx.x] = a;
        }
    }
    if (!counters || nsplit == 1) return;  // a separate merge kernel follows / nothing to merge
    // The last split of this (sequence, head) to finish merges all partial records: publish
    // ours, count arrivals, and only the final arriver reads the others back.
    // The record stores above are device-scope (write-through) and have completed before the
    // barrier below releases thread 0, so a relaxed device-scope counter is enough; a full
    // release fence here would write back the whole L2 (measured: 12x slower kernel).
    __shared__ uint32_t is_last;
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t prev = __hip_atomic_fetch_add(counters + b * heads + h, 1u, __ATOMIC_RELAXED,
                                                     __HIP_MEMORY_SCOPE_AGENT);
        is_last = prev == nsplit - 1;
        if (is_last)  // ready for the next launch
            __hip_atomic_store(counters + b * heads + h, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!is_last) return;
    // All records are fetched with independent loads by the whole workgroup (a loop of
    // dependent device-scope loads would pay the L2 latency once per split), then merged from LDS.
    const float *rec_g = part + ((uint64_t)b * heads + h) * nsplit * (HD + 2);
    const uint32_t nrec = nsplit * (HD + 2);
    for (uint32_t i0 = 0; i0 < nrec; i0 += 4 * NW * 64) {
        float tmp[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const uint32_t i = i0 + u * NW * 64 + threadIdx.x;
            tmp[u] = i < nrec ? __hip_atomic_load(rec_g + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0.f;
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const uint32_t i = i0 + u * NW * 64 + threadIdx.x;
            if (i < nrec) srec[i] = tmp[u];
        }
    }
    __syncthreads();
    if (threadIdx.x < HD) {
        const float *rec = srec;
        float mm = -INFINITY;
        for (uint32_t s2 = 0; s2 < nsplit; s2++) mm = fmaxf(mm, rec[s2 * (HD + 2)]);
        float lt = 0.f, a = 0.f;
        for (uint32_t s2 = 0; s2 < nsplit; s2++) {
            const float ms = rec[s2 * (HD + 2)];
            const float c = ms == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms - mm);
            lt += rec[s2 * (HD + 2) + 1] * c;
            a += rec[s2 * (HD + 2) + 2 + threadIdx.x] * c;
        }
        const float r = a / lt;
        if (out) out[(uint64_t)b * inner + h * HD + threadIdx.x] = r;
        if (out_xq) out_xq[xq_index(h * HD + threadIdx.x, b, bp)] = __float2half_rn(r);
    }
}

template <int HD>
__global__ void attn_merge_kernel(const float *__restrict__ part, uint32_t heads, uint32_t nsplit,
                                  float *out, __half *out_xq, uint32_t bp) {
    const uint32_t h = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
    const float *rec = part + ((uint64_t)b * heads + h) * nsplit * (HD + 2);
    float mm = -INFINITY;
    for (uint32_t s = 0; s < nsplit; s++) mm = fmaxf(mm, rec[s * (HD + 2)]);
    float lt = 0.f, a = 0.f;
    for (uint32_t s = 0; s < nsplit; s++) {
        const float ms = rec[s * (HD + 2)];
        const float c = ms == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms - mm);  // (the records' maxima are in base 2)
        lt += rec[s * (HD + 2) + 1] * c;
        a += rec[s * (HD + 2) + 2 + d] * c;
    }
    const float r = a / lt;
    const uint32_t inner = heads * HD;
    if (out) out[(uint64_t)b * inner + h * HD + d] = r;
    if (out_xq) out_xq[xq_index(h * HD + d, b, bp)] = __float2half_rn(r);
}

// ---------------------------------------------------------------- launchers
// ---------------------------------------------------------------- prefill on the matrix cores
// One workgroup per (128 query rows, head, sequence), 4 waves of 32 query rows; keys in tiles of
// 32, double-buffered in LDS.  Both products are computed transposed so that a query stays in
// the same lanes from the scores to the output and the probabilities never leave registers:
//   S^T[key][q] = K . Q^T   (A = K tile rows from LDS, B = the wave's Q fragments, in registers
//                            for the whole kernel): lane l holds query l % 32 and 16 keys
//   O^T[d][q]  += V^T . P^T (A = V^T from LDS, B = P^T = exp(S^T - max) packed to 16 bit)
// A matrix-core reduction index is only a summation label, so the 16 keys a lane holds
// (8g + 4*(l/32) + 0..3, g = 0..3) are fed to P.V in that order, and the V tile is transposed
// into LDS as [dim][key] on the way in, so the matching V^T operand is two 8-byte reads.
// The row max needs one cross-lane step per tile (lanes l and l + 32 share a query; a register
// swap, not a trip through LDS); the row sum is kept per lane and the two halves are added once,
// after the loop.
// Within a wave a key tile is a strict chain (scores -> softmax on the VALU -> P.V), so the
// matrix cores are only kept busy by other waves of the SIMD: the register budget is capped at
// what lets three workgroups share a CU (measured: 17 % faster than two).
// Which (query tile, head) a workgroup of a prefill grid (x = query tiles, y = heads) works on.
// Causal work grows with the query tile: the last (longest) tiles are dispatched first, so that
// the short ones fill in behind them instead of the long ones forming the tail.  The hardware
// deals consecutive workgroups round-robin to the 8 XCDs: with a multiple of 8 heads the numbering
// is permuted so that all query tiles of a head run on one XCD and its keys and values are fetched
// into one L2 instead of eight (measured on 32 heads x 4024 rows: 292 -> 184 us).
__device__ __forceinline__ void prefill_tile_of_block(uint32_t &qt, uint32_t &h) {
    qt = gridDim.x - 1 - blockIdx.x;
    h = blockIdx.y;
    if ((gridDim.y & 7) == 0) {
        const uint32_t lin = blockIdx.x + gridDim.x * blockIdx.y, idx = lin >> 3, hpx = gridDim.y >> 3;
        h = (lin & 7) + 8 * (idx % hpx);
        qt = gridDim.x - 1 - idx / hpx;
    }
}

// Maximum of a value over lanes i and i ^ 32 (v_permlane32_swap hands every lane both values: a
// register move, no trip through LDS); the sum is xor32_sum.
__device__ __forceinline__ float both_halves_max(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

template <int HD, bool BF16>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 4))) void attn_prefill_kernel(const float *__restrict__ qkv,
                                                           const uint16_t *__restrict__ kc,
                                                           const uint16_t *__restrict__ vc,
                                                           uint32_t n, uint32_t heads,
                                                           uint32_t max_ctx, uint32_t pos0,
                                                           float *__restrict__ out,
                                                           uint16_t *__restrict__ out_lp,
                                                           uint64_t lp_ld, bool lp_bf16) {
    constexpr int KT = 32, KLD = HD + 8, VLD = 36, NKS = HD / 16, NDT = HD / 32;
    __shared__ __attribute__((aligned(16))) uint16_t ks[2][KT * KLD];  // [key][dim]
    __shared__ __attribute__((aligned(16))) uint16_t vt[2][HD * VLD];  // [dim][key]
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t qi = lane & 31, hf = lane >> 5;
    uint32_t qt, h;
    prefill_tile_of_block(qt, h);
    const uint32_t b = blockIdx.z;
    const uint32_t inner = heads * HD;
    const uint32_t r0 = qt * 128 + wave * 32;          // the wave's first query row
    const uint32_t r = r0 + qi, rc = r < n ? r : n - 1;  // rows past the end repeat the last
    const uint32_t qpos = pos0 + rc;
    const float scale2 = 1.4426950408889634f / sqrtf((float)HD);  // scale * log2(e)

    auto pack2 = [](float a, float c) -> uint32_t {
        if (BF16) return (uint32_t)f32_to_bf16_bits(a) | ((uint32_t)f32_to_bf16_bits(c) << 16);
        union { half2_t h; uint32_t u; } cv;
        cv.h.x = (_Float16)a; cv.h.y = (_Float16)c;
        return cv.u;
    };
    // Q fragments: query rc, dims 16 ks + 8 hf .. + 7
    uint4 qf[NKS];
    {
        const float *qp = qkv + ((uint64_t)b * n + rc) * 3 * inner + h * HD + 8 * hf;
#pragma unroll
        for (int s = 0; s < NKS; s++) {
            const float4 a = *(const float4 *)(qp + 16 * s), c = *(const float4 *)(qp + 16 * s + 4);
            qf[s] = make_uint4(pack2(a.x, a.y), pack2(a.z, a.w), pack2(c.x, c.y), pack2(c.z, c.w));
        }
    }
    const uint64_t base = ((uint64_t)b * heads + h) * max_ctx * HD;
    const uint16_t *kb = kc + base, *vb = vc + base;
    const uint32_t q_hi = min(n, qt * 128 + 128) - 1;   // last query row of the workgroup
    const uint32_t kmax = pos0 + q_hi;                  // last key any of its rows attends to
    const uint32_t ntiles = kmax / KT + 1;
    const uint32_t wave_kmax = pos0 + min(n - 1, r0 + 31);  // (waves past the end do no work)
    const bool wave_live = r0 < n;

    // global -> registers -> LDS.  K: thread t takes 16-byte pieces t % 8 (+ 8) of key t / 8.
    // V: thread t takes piece t / 16 of keys 2 (t % 16) and 2 (t % 16) + 1 and stores them
    // interleaved, one dword = the two keys of one dim.
    const uint32_t kkey = tid >> 3, kpc = tid & 7, vc2 = tid & 15, vdp = tid >> 4;
    uint4 rk0, rk1, rv0, rv1;
    auto gload = [&](uint32_t t) {
        const uint32_t key = min(t * KT + kkey, kmax);  // keys past the last one repeat it (finite values)
        // (a head's slab of the cache is below 4 GiB: 32-bit offsets from a uniform base)
        rk0 = *(const uint4 *)(kb + (key * HD + kpc * 8));
        if (HD == 128) rk1 = *(const uint4 *)(kb + (key * HD + 64 + kpc * 8));
        if (HD == 128 || vdp < 8) {
            const uint32_t k0 = min(t * KT + 2 * vc2, kmax), k1 = min(t * KT + 2 * vc2 + 1, kmax);
            rv0 = *(const uint4 *)(vb + (k0 * HD + vdp * 8));
            rv1 = *(const uint4 *)(vb + (k1 * HD + vdp * 8));
        }
    };
    auto lstore = [&](uint32_t buf) {
        *(uint4 *)(&ks[buf][kkey * KLD + kpc * 8]) = rk0;
        if (HD == 128) *(uint4 *)(&ks[buf][kkey * KLD + 64 + kpc * 8]) = rk1;
        if (HD == 128 || vdp < 8) {
            const uint32_t a[4] = {rv0.x, rv0.y, rv0.z, rv0.w}, c[4] = {rv1.x, rv1.y, rv1.z, rv1.w};
            // one base address; the eight rows differ by constants (immediate offsets of the stores)
            uint32_t *dst = (uint32_t *)&vt[buf][0] + vdp * (8 * VLD / 2) + vc2;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                // dims 8 vdp + 2e, + 2e + 1: low halves / high halves of the two keys
                dst[e * VLD] = __builtin_amdgcn_perm(c[e], a[e], 0x05040100u);
                dst[e * VLD + VLD / 2] = __builtin_amdgcn_perm(c[e], a[e], 0x07060302u);
            }
        }
    };

    float16_t o[NDT];
#pragma unroll
    for (int d = 0; d < NDT; d++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[d][i] = 0.f;
    float m = -INFINITY, l = 0.f;

    gload(0);
    lstore(0);
    gload(ntiles > 1 ? 1 : 0);
    for (uint32_t t = 0; t < ntiles; t++) {
        __syncthreads();  // tile t is in LDS; everybody is done with the buffer of tile t - 1
        lstore((t + 1) & 1);                       // tile t + 1 (requested one tile ago)
        gload(t + 2 < ntiles ? t + 2 : ntiles - 1);  // unconditional; the repeat is never used
        if (!wave_live || t * KT > wave_kmax) continue;  // wave-uniform: nothing left to attend to
        const uint16_t *kt_ = ks[t & 1], *vt_ = vt[t & 1];
        // scores, transposed: lane = query qi; element i = key 8 (i / 4) + 4 hf + i % 4
        float16_t sc;
#pragma unroll
        for (int i = 0; i < 16; i++) sc[i] = 0.f;
#pragma unroll
        for (int s = 0; s < NKS; s++) {
            const uint4 kf = *(const uint4 *)(kt_ + qi * KLD + 16 * s + 8 * hf);
            if (BF16) {
                union { uint4 u; bf16x8_t v; } ua, ub;
                ua.u = kf; ub.u = qf[s];
                sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ua.v, ub.v, sc, 0, 0, 0);
            } else {
                union { uint4 u; half8_t v; } ua, ub;
                ua.u = kf; ub.u = qf[s];
                sc = __builtin_amdgcn_mfma_f32_32x32x16_f16(ua.v, ub.v, sc, 0, 0, 0);
            }
        }
        // Online softmax in base 2: with c = scale * log2(e), p = 2^(c s - m) where m is the
        // running maximum of c s; one fused multiply-add and one v_exp_f32 per score.
        const uint32_t key0 = t * KT + 4 * hf;
        const bool diag = t * KT + KT - 1 > pos0 + r0;  // some (query, key) pair of the tile is masked
        float tmax = -INFINITY;
        if (diag) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const uint32_t key = key0 + 8 * (i >> 2) + (i & 3);
                sc[i] = key > qpos ? -INFINITY : sc[i];
            }
        }
#pragma unroll
        for (int i = 0; i < 16; i++) tmax = fmaxf(tmax, sc[i]);
        tmax = both_halves_max(tmax) * scale2;  // scale2 > 0: max commutes with it
        const float m_new = fmaxf(m, tmax);  // finite: key 0 is never masked
        float psum = 0.f;
        float pv[16];
#pragma unroll
        for (int i = 0; i < 16; i++) {
            pv[i] = __builtin_amdgcn_exp2f(fmaf(sc[i], scale2, -m_new));  // 2^(-inf) = 0 for masked keys
            psum += pv[i];
        }
        // the accumulators are rescaled only when some query of the wave got a new maximum
        if (__builtin_amdgcn_ballot_w64(m_new != m) != 0) {
            const float corr = __builtin_amdgcn_exp2f(m - m_new);
            l *= corr;
#pragma unroll
            for (int d = 0; d < NDT; d++)
#pragma unroll
                for (int i = 0; i < 16; i++) o[d][i] *= corr;
        }
        l += psum;
        m = m_new;
        // P^T operands: reduction slot (hf, e) of instruction j <-> key 8 (2j + e / 4) + 4 hf + e % 4
        uint4 pf[2];
#pragma unroll
        for (int j = 0; j < 2; j++)
            pf[j] = make_uint4(pack2(pv[8 * j], pv[8 * j + 1]), pack2(pv[8 * j + 2], pv[8 * j + 3]),
                               pack2(pv[8 * j + 4], pv[8 * j + 5]), pack2(pv[8 * j + 6], pv[8 * j + 7]));
#pragma unroll
        for (int d = 0; d < NDT; d++)
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const uint16_t *vp = vt_ + (d * 32 + qi) * VLD + 16 * j + 4 * hf;
                const uint2 v0 = *(const uint2 *)vp, v1 = *(const uint2 *)(vp + 8);
                const uint4 vf = make_uint4(v0.x, v0.y, v1.x, v1.y);
                if (BF16) {
                    union { uint4 u; bf16x8_t v; } ua, ub;
                    ua.u = vf; ub.u = pf[j];
                    o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ua.v, ub.v, o[d], 0, 0, 0);
                } else {
                    union { uint4 u; half8_t v; } ua, ub;
                    ua.u = vf; ub.u = pf[j];
                    o[d] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ua.v, ub.v, o[d], 0, 0, 0);
                }
            }
    }
    if (r >= n) return;
    const float inv = 1.0f / xor32_sum(l);
    if (out) {
        float *op = out + ((uint64_t)b * n + r) * inner + h * HD + 4 * hf;
#pragma unroll
        for (int d = 0; d < NDT; d++)
#pragma unroll
            for (int g = 0; g < 4; g++)
                *(float4 *)(op + d * 32 + 8 * g) = make_float4(o[d][4 * g] * inv, o[d][4 * g + 1] * inv,
                                                               o[d][4 * g + 2] * inv, o[d][4 * g + 3] * inv);
    }
    if (out_lp) {  // 16-bit rows for the output projection's A operand
        uint16_t *op = out_lp + ((uint64_t)b * n + r) * lp_ld + h * HD + 4 * hf;
#pragma unroll
        for (int d = 0; d < NDT; d++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                uint2 v;
                v.x = (uint32_t)f32_to_lp_bits(o[d][4 * g] * inv, lp_bf16) | ((uint32_t)f32_to_lp_bits(o[d][4 * g + 1] * inv, lp_bf16) << 16);
                v.y = (uint32_t)f32_to_lp_bits(o[d][4 * g + 2] * inv, lp_bf16) | ((uint32_t)f32_to_lp_bits(o[d][4 * g + 3] * inv, lp_bf16) << 16);
                *(uint2 *)(op + d * 32 + 8 * g) = v;
            }
    }
}

// ---------------------------------------------------------------- prefill, f32 cache
// The same scheme on the f32 matrix-core instruction (v_mfma_f32_32x32x2_f32), for models that
// keep the reference's f32 keys and values: every operand and every product stays f32.
//   S^T[key][q] = K . Q^T: instruction s sums over the two dims {s, HD/2 + s} (a reduction index is
//       only a label): lane l = (row l % 32, half l / 32) feeds K[key l%32][half*HD/2 + s] from LDS
//       and Q[query l%32][half*HD/2 + s] from registers.
//   O^T[d][q] += V^T . P^T: instruction j sums over the two keys 8(j/4) + j%4 and that + 4, which are
//       exactly the keys whose probabilities element j of the two lane halves holds; the V operand
//       is one LDS dword per lane (V[key][d], lanes along d).
template <int HD>
__global__ __launch_bounds__(256) void attn_prefill_f32_kernel(const float *__restrict__ qkv,
                                                               const float *__restrict__ kc,
                                                               const float *__restrict__ vc,
                                                               uint32_t n, uint32_t heads,
                                                               uint32_t max_ctx, uint32_t pos0,
                                                               float *__restrict__ out) {
    constexpr int KT = 32, LD = HD + 4, HH = HD / 2, NDT = HD / 32;
    constexpr int PCS = KT * HD / 4 / 256;  // float4 pieces of a tile per thread (2 or 4)
    __shared__ __attribute__((aligned(16))) float ks[2][KT * LD];  // [key][dim]
    __shared__ __attribute__((aligned(16))) float vs[2][KT * LD];  // [key][dim]
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t qi = lane & 31, hf = lane >> 5;
    uint32_t qt, h;
    prefill_tile_of_block(qt, h);  // longest first, a head's tiles on one XCD
    const uint32_t b = blockIdx.z;
    const uint32_t inner = heads * HD;
    const uint32_t r0 = qt * 128 + wave * 32;
    const uint32_t r = r0 + qi, rc = r < n ? r : n - 1;  // rows past the end repeat the last
    const uint32_t qpos = pos0 + rc;
    const float scale2 = 1.4426950408889634f / sqrtf((float)HD);  // scale * log2(e)

    float qf[HH];
    {
        const float *qp = qkv + ((uint64_t)b * n + rc) * 3 * inner + h * HD + hf * HH;
#pragma unroll
        for (int s = 0; s < HH; s += 4) {
            const float4 a = *(const float4 *)(qp + s);
            qf[s] = a.x; qf[s + 1] = a.y; qf[s + 2] = a.z; qf[s + 3] = a.w;
        }
    }
    const uint64_t base = ((uint64_t)b * heads + h) * max_ctx * HD;
    const float *kb = kc + base, *vb = vc + base;
    const uint32_t q_hi = min(n, qt * 128 + 128) - 1;
    const uint32_t kmax = pos0 + q_hi;  // last key any row of the workgroup attends to
    const uint32_t ntiles = kmax / KT + 1;
    const uint32_t wave_kmax = pos0 + min(n - 1, r0 + 31);
    const bool wave_live = r0 < n;

    // global -> registers -> LDS: piece p = tid + 256 u is float4 (p % (HD/4)) of key p / (HD/4).
    // (Named registers, not arrays: arrays captured by these lambdas end up in scratch memory.)
    float4 rk0, rk1, rk2, rk3, rv0, rv1, rv2, rv3;
    rk2 = rk3 = rv2 = rv3 = make_float4(0.f, 0.f, 0.f, 0.f);
    auto gload1 = [&](uint32_t t, uint32_t u, float4 &k4, float4 &v4) {
        const uint32_t p = tid + 256 * u, key = min(t * KT + p / (HD / 4), kmax), c = p % (HD / 4);
        k4 = *(const float4 *)(kb + (uint64_t)key * HD + 4 * c);
        v4 = *(const float4 *)(vb + (uint64_t)key * HD + 4 * c);
    };
    auto lstore1 = [&](uint32_t buf, uint32_t u, const float4 &k4, const float4 &v4) {
        const uint32_t p = tid + 256 * u, kk = p / (HD / 4), c = p % (HD / 4);
        *(float4 *)(&ks[buf][kk * LD + 4 * c]) = k4;
        *(float4 *)(&vs[buf][kk * LD + 4 * c]) = v4;
    };
    auto gload = [&](uint32_t t) {
        gload1(t, 0, rk0, rv0);
        gload1(t, 1, rk1, rv1);
        if (PCS > 2) { gload1(t, 2, rk2, rv2); gload1(t, 3, rk3, rv3); }
    };
    auto lstore = [&](uint32_t buf) {
        lstore1(buf, 0, rk0, rv0);
        lstore1(buf, 1, rk1, rv1);
        if (PCS > 2) { lstore1(buf, 2, rk2, rv2); lstore1(buf, 3, rk3, rv3); }
    };

    float16_t o[NDT];
#pragma unroll
    for (int d = 0; d < NDT; d++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[d][i] = 0.f;
    float m = -INFINITY, l = 0.f;

    gload(0);
    lstore(0);
    gload(ntiles > 1 ? 1 : 0);
    for (uint32_t t = 0; t < ntiles; t++) {
        __syncthreads();  // tile t is in LDS; everybody is done with the buffer of tile t - 1
        lstore((t + 1) & 1);
        gload(t + 2 < ntiles ? t + 2 : ntiles - 1);
        if (!wave_live || t * KT > wave_kmax) continue;  // wave-uniform
        const float *kt_ = ks[t & 1], *vt_ = vs[t & 1];
        float16_t sc;
#pragma unroll
        for (int i = 0; i < 16; i++) sc[i] = 0.f;
#pragma unroll
        for (int s4 = 0; s4 < HH; s4 += 4) {
            const float4 kf = *(const float4 *)(kt_ + qi * LD + hf * HH + s4);
            sc = __builtin_amdgcn_mfma_f32_32x32x2f32(kf.x, qf[s4], sc, 0, 0, 0);
            sc = __builtin_amdgcn_mfma_f32_32x32x2f32(kf.y, qf[s4 + 1], sc, 0, 0, 0);
            sc = __builtin_amdgcn_mfma_f32_32x32x2f32(kf.z, qf[s4 + 2], sc, 0, 0, 0);
            sc = __builtin_amdgcn_mfma_f32_32x32x2f32(kf.w, qf[s4 + 3], sc, 0, 0, 0);
        }
        // online softmax in base 2 (see attn_prefill_kernel); element i = key 8 (i / 4) + 4 hf + i % 4
        const uint32_t key0 = t * KT + 4 * hf;
        const bool diag = t * KT + KT - 1 > pos0 + r0;
        if (diag) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const uint32_t key = key0 + 8 * (i >> 2) + (i & 3);
                sc[i] = key > qpos ? -INFINITY : sc[i];
            }
        }
        float tmax = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; i++) tmax = fmaxf(tmax, sc[i]);
        tmax = both_halves_max(tmax) * scale2;
        const float m_new = fmaxf(m, tmax);  // finite: key 0 is never masked
        float psum = 0.f, pv[16];
#pragma unroll
        for (int i = 0; i < 16; i++) {
            pv[i] = __builtin_amdgcn_exp2f(fmaf(sc[i], scale2, -m_new));
            psum += pv[i];
        }
        psum = xor32_sum(psum);
        if (__builtin_amdgcn_ballot_w64(m_new != m) != 0) {
            const float corr = __builtin_amdgcn_exp2f(m - m_new);
            l *= corr;
#pragma unroll
            for (int d = 0; d < NDT; d++)
#pragma unroll
                for (int i = 0; i < 16; i++) o[d][i] *= corr;
        }
        l += psum;
        m = m_new;
#pragma unroll
        for (int j = 0; j < 16; j++) {
            const uint32_t key = 8 * (j >> 2) + 4 * hf + (j & 3);
#pragma unroll
            for (int d = 0; d < NDT; d++)
                o[d] = __builtin_amdgcn_mfma_f32_32x32x2f32(vt_[key * LD + d * 32 + qi], pv[j], o[d], 0, 0, 0);
        }
    }
    if (r >= n) return;
    const float inv = 1.0f / l;
    float *op = out + ((uint64_t)b * n + r) * inner + h * HD + 4 * hf;
#pragma unroll
    for (int d = 0; d < NDT; d++)
#pragma unroll
        for (int g = 0; g < 4; g++)
            *(float4 *)(op + d * 32 + 8 * g) = make_float4(o[d][4 * g] * inv, o[d][4 * g + 1] * inv,
                                                           o[d][4 * g + 2] * inv, o[d][4 * g + 3] * inv);
}

int launch_kv_append(const float *qkv, void *kc, void *vc, uint32_t kv_dtype, uint64_t batch,
                     uint64_t n, uint64_t heads, uint64_t hd, uint64_t max_ctx, uint64_t pos0,
                     const uint32_t *pos_dev, hipStream_t st) {
    const dim3 grid((unsigned)(batch * n)), block(256);
#define COEUS_KVA(T)                                                                              \
    hipLaunchKernelGGL(kv_append_kernel<T>, grid, block, 0, st, qkv, (T *)kc, (T *)vc, (uint32_t)n, \
                       (uint32_t)heads, (uint32_t)hd, (uint32_t)max_ctx, (uint32_t)pos0, pos_dev)
    if (kv_dtype == COEUS_KV_F32) COEUS_KVA(float);
    else if (kv_dtype == COEUS_KV_F16) COEUS_KVA(__half);
    else COEUS_KVA(uint16_t);
#undef COEUS_KVA
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

bool attn_prefill_on_matrix_cores(uint64_t n, uint64_t hd, uint32_t kv_dtype) {
    return n >= 16 && (hd == 64 || hd == 128) && kv_dtype != COEUS_KV_F32;
}

uint32_t attn_decode_splits(uint64_t batch, uint64_t heads, uint64_t max_ctx) {
    // Aim for one workgroup per CU, at least 256 keys per split.  Measured at context 4096 with 32
    // heads of 128: batch 1, 8 splits 17.3 us against 17.8 with 16; batch 4, 2 splits 46.3 us
    // against 49.0 with 8; batch 16, 1 split 182.7 us against 187.9 with 2 (fewer partial records
    // to publish and merge; the kernel's two workgroups per CU stream at the same rate either way).
    // A power of two: three splits of 2048 keys (704 + 704 + 640, the wave tiles no longer line up)
    // ran 17.6 us at batch 8 x 12 heads of 64 against 14.0 us with four.
    uint64_t want = ceil_div(256, batch * heads);
    while (want & (want - 1)) want++;  // up to the next power of two
    uint64_t cap = ceil_div(max_ctx, 256);
    uint64_t s = 1;
    while (s * 2 <= want && s * 2 <= cap && s * 2 <= kAttnMaxSplits) s *= 2;
    return (uint32_t)s;
}

int launch_attention(const float *qkv, const void *kc, const void *vc, uint32_t kv_dtype,
                     uint64_t batch, uint64_t n, uint64_t heads, uint64_t hd, uint64_t max_ctx,
                     uint64_t pos0, const uint32_t *pos_dev, float *out, __half *out_xq,
                     uint32_t bp, float *part_scratch, uint32_t nsplit, uint32_t *counters,
                     hipStream_t st, const LpOut *out_lp) {
    if (hd == 0 || hd > 256) return fail(COEUS_INVALID_INPUT, "head_dim %llu out of range [1, 256]",
                                         (unsigned long long)hd);
    // the kernels index a head's slab of the cache with 32 bits
    if (max_ctx * hd > 0xffffffffull)
        return fail(COEUS_INVALID_INPUT, "attention: max_ctx %llu x head_dim %llu exceeds 2^32 elements per head",
                    (unsigned long long)max_ctx, (unsigned long long)hd);
    const bool fast = n == 1 && (hd == 64 || hd == 128) && kv_dtype != COEUS_KV_F32 &&
                      part_scratch && nsplit >= 1;
    if (fast) {
        if (counters && nsplit > kAttnMaxSplits)
            return fail(COEUS_INVALID_INPUT, "attention: at most %u splits with the in-kernel merge",
                        kAttnMaxSplits);
        const uint32_t kps = (uint32_t)round_up(ceil_div(max_ctx, nsplit), 64);
        const dim3 grid(nsplit, (unsigned)heads, (unsigned)batch);
        const bool bf = kv_dtype == COEUS_KV_BF16;
        // One workgroup per CU at most and splits of 512 keys or more: 8 waves per workgroup, a tile
        // of 64 keys each at once, instead of 4 waves walking two tiles each (7B shape, batch 1,
        // context 4096: 1.768 -> 1.759 ms per step over five alternations; with shorter splits the
        // extra waves have nothing to take and the step is 0.5 % slower).
        const bool wide = batch * heads * nsplit <= 256 && kps >= 512;
#define COEUS_AD(HDV, BFV) do {                                                                    \
    if (wide)                                                                                      \
    hipLaunchKernelGGL((attn_decode_kernel<HDV, BFV, 8>), grid, dim3(512), 0, st, qkv,             \
                       (const uint16_t *)kc, (const uint16_t *)vc, (uint32_t)heads,                \
                       (uint32_t)max_ctx, (uint32_t)pos0, pos_dev, kps, part_scratch, counters,    \
                       out, out_xq, bp);                                                           \
    else                                                                                           \
    hipLaunchKernelGGL((attn_decode_kernel<HDV, BFV>), grid, dim3(256), 0, st, qkv,                \
                       (const uint16_t *)kc, (const uint16_t *)vc, (uint32_t)heads,                \
                       (uint32_t)max_ctx, (uint32_t)pos0, pos_dev, kps, part_scratch, counters,    \
                       out, out_xq, bp); } while (0)
        if (hd == 64) { if (bf) COEUS_AD(64, true); else COEUS_AD(64, false); }
        else { if (bf) COEUS_AD(128, true); else COEUS_AD(128, false); }
#undef COEUS_AD
        COEUS_HIP(hipGetLastError());
        if (counters || nsplit == 1) return COEUS_OK;  // merged by the last split of each (sequence, head)
        const dim3 mg((unsigned)heads, (unsigned)batch);
        if (hd == 64)
            hipLaunchKernelGGL(attn_merge_kernel<64>, mg, dim3(64), 0, st, part_scratch, (uint32_t)heads, nsplit, out, out_xq, bp);
        else
            hipLaunchKernelGGL(attn_merge_kernel<128>, mg, dim3(128), 0, st, part_scratch, (uint32_t)heads, nsplit, out, out_xq, bp);
        COEUS_HIP(hipGetLastError());
        return COEUS_OK;
    }
    uint16_t *lp = out_lp ? (uint16_t *)out_lp->p : nullptr;
    const uint64_t lp_ld = out_lp ? out_lp->ld : 0;
    const bool lp_bf = out_lp && out_lp->bf16;
    if (attn_prefill_on_matrix_cores(n, hd, kv_dtype) && !pos_dev && (out || lp) && !out_xq) {
        const dim3 pgrid((unsigned)ceil_div(n, 128), (unsigned)heads, (unsigned)batch);
        const bool bf = kv_dtype == COEUS_KV_BF16;
#define COEUS_AP(HDV, BFV)                                                                         \
    hipLaunchKernelGGL((attn_prefill_kernel<HDV, BFV>), pgrid, dim3(256), 0, st, qkv,              \
                       (const uint16_t *)kc, (const uint16_t *)vc, (uint32_t)n, (uint32_t)heads,   \
                       (uint32_t)max_ctx, (uint32_t)pos0, out, lp, lp_ld, lp_bf)
        if (hd == 64) { if (bf) COEUS_AP(64, true); else COEUS_AP(64, false); }
        else { if (bf) COEUS_AP(128, true); else COEUS_AP(128, false); }
#undef COEUS_AP
        COEUS_HIP(hipGetLastError());
        return COEUS_OK;
    }
    if (lp) return fail(COEUS_INVALID_INPUT, "16-bit attention output needs the matrix-core prefill kernel");
    if (kv_dtype == COEUS_KV_F32 && n >= 16 && (hd == 64 || hd == 128) && !pos_dev && out && !out_xq) {
        const dim3 pgrid((unsigned)ceil_div(n, 128), (unsigned)heads, (unsigned)batch);
        if (hd == 64)
            hipLaunchKernelGGL(attn_prefill_f32_kernel<64>, pgrid, dim3(256), 0, st, qkv, (const float *)kc,
                               (const float *)vc, (uint32_t)n, (uint32_t)heads, (uint32_t)max_ctx,
                               (uint32_t)pos0, out);
        else
            hipLaunchKernelGGL(attn_prefill_f32_kernel<128>, pgrid, dim3(256), 0, st, qkv, (const float *)kc,
                               (const float *)vc, (uint32_t)n, (uint32_t)heads, (uint32_t)max_ctx,
                               (uint32_t)pos0, out);
        COEUS_HIP(hipGetLastError());
        return COEUS_OK;
    }
    const dim3 grid((unsigned)ceil_div(n, 4), (unsigned)heads, (unsigned)batch);
    const size_t lds = 4 * (hd + 64) * sizeof(float);
#define COEUS_AG(T)                                                                                 \
    hipLaunchKernelGGL(attn_generic_kernel<T>, grid, dim3(256), lds, st, qkv, (const T *)kc,        \
                       (const T *)vc, (uint32_t)n, (uint32_t)heads, (uint32_t)hd, (uint32_t)max_ctx, \
                       (uint32_t)pos0, pos_dev, out, out_xq, bp)
    if (kv_dtype == COEUS_KV_F32) COEUS_AG(float);
    else if (kv_dtype == COEUS_KV_F16) COEUS_AG(__half);
    else COEUS_AG(uint16_t);
#undef COEUS_AG
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

}  // namespace coeus
