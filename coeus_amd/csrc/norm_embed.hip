// Normalisation, embedding gather and small element-wise kernels.
//
//   norm_token_kernel     one workgroup per row: LayerNorm / RMSNorm with per-row statistics.
//   norm_rows_kernel      the same for many rows of up to 1024 elements: one wave per row.
//   norm_sequence_kernel  math::layer_norm exactly as the reference calls it (MT:105-128 from
//                         MT:469,488,906): ONE mean/variance over the whole [rows*hidden] slice,
//                         scale/bias indexed i % hidden.
//   embed_kernel          x[s,:] = E[id_s,:] + PE[pos0+s,:]  (MT:812-835)
#include "device_utils.hpp"

namespace coeus {

__device__ __forceinline__ float block_sum(float v, float *sh) {
    // blockDim.x <= 1024; sh holds 16 floats
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) sh[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (uint32_t w = 0; w < nw; w++) t += sh[w];
    return t;
}

__device__ __forceinline__ double block_sum_f64(double v, double *sh) {
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    __syncthreads();
    if (lane == 0) sh[wave] = v;
    __syncthreads();
    double t = 0.0;
    for (uint32_t w = 0; w < nw; w++) t += sh[w];
    return t;
}

// y = scale * (x - mean) / sqrt(var + eps) + bias (MT:124: (scale * (x - mean)) / std + bias); rows
// of a multiple of 4 elements multiply by 1 / std instead of dividing.
template <bool RMS>
__global__ __launch_bounds__(256) void norm_token_kernel(const float *__restrict__ x, uint64_t hidden,
                                                         const float *__restrict__ scale,
                                                         const float *__restrict__ bias, float eps,
                                                         float *y, __half *y_xq, uint32_t bp,
                                                         uint16_t *y_lp, uint64_t lp_ld, bool lp_bf16) {
    __shared__ float sh[16];
    const uint64_t row = blockIdx.x;
    const float *xr = x + row * hidden;
    // rows of up to 8192 elements (a multiple of 4) are read once, 16 bytes per lane at a time,
    // and kept in registers for both statistics passes and the final pass
    constexpr int VMAX = 8;
    const bool fast = (hidden & 3) == 0 && hidden <= 4u * 256u * VMAX && (lp_ld & 3) == 0;
    if (fast) {
        const uint32_t n4 = (uint32_t)(hidden / 4);
        float4 v[VMAX];
#pragma unroll
        for (int u = 0; u < VMAX; u++) {
            const uint32_t i = threadIdx.x + 256 * u;
            v[u] = i < n4 ? *(const float4 *)(xr + 4 * i) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
        float mean = 0.f;
        if (!RMS) {
            float s = 0.f;
#pragma unroll
            for (int u = 0; u < VMAX; u++) s += (v[u].x + v[u].y) + (v[u].z + v[u].w);
            mean = block_sum(s, sh) / (float)hidden;
        }
        float s2 = 0.f;
#pragma unroll
        for (int u = 0; u < VMAX; u++) {
            if (threadIdx.x + 256 * u < n4) {
                const float d0 = v[u].x - mean, d1 = v[u].y - mean, d2 = v[u].z - mean, d3 = v[u].w - mean;
                s2 = fmaf(d0, d0, s2); s2 = fmaf(d1, d1, s2); s2 = fmaf(d2, d2, s2); s2 = fmaf(d3, d3, s2);
            }
        }
        const float var = block_sum(s2, sh) / (float)hidden;
        // one division per row; the elements are multiplied by the reciprocal (an ulp from the
        // reference's (scale * (x - mean)) / std, and a third of this kernel's instructions less)
        const float rs = 1.0f / sqrtf(var + eps);
#pragma unroll
        for (int u = 0; u < VMAX; u++) {
            const uint32_t i = threadIdx.x + 256 * u;
            if (i >= n4) continue;
            const float4 sc = *(const float4 *)(scale + 4 * i);
            float o[4] = {sc.x * (v[u].x - mean) * rs, sc.y * (v[u].y - mean) * rs,
                          sc.z * (v[u].z - mean) * rs, sc.w * (v[u].w - mean) * rs};
            if (!RMS) {
                const float4 bi = *(const float4 *)(bias + 4 * i);
                o[0] += bi.x; o[1] += bi.y; o[2] += bi.z; o[3] += bi.w;
            }
            if (y) *(float4 *)(y + row * hidden + 4 * i) = make_float4(o[0], o[1], o[2], o[3]);
            if (y_xq) {
#pragma unroll
                for (int q = 0; q < 4; q++) y_xq[xq_index(4 * i + q, (uint32_t)row, bp)] = __float2half_rn(o[q]);
            }
            if (y_lp) {
                uint2 p;
                p.x = (uint32_t)f32_to_lp_bits(o[0], lp_bf16) | ((uint32_t)f32_to_lp_bits(o[1], lp_bf16) << 16);
                p.y = (uint32_t)f32_to_lp_bits(o[2], lp_bf16) | ((uint32_t)f32_to_lp_bits(o[3], lp_bf16) << 16);
                *(uint2 *)(y_lp + row * lp_ld + 4 * i) = p;
            }
        }
        return;
    }
    float mean = 0.f;
    if (!RMS) {
        float s = 0.f;
        for (uint64_t i = threadIdx.x; i < hidden; i += blockDim.x) s += xr[i];
        mean = block_sum(s, sh) / (float)hidden;
    }
    float s2 = 0.f;
    for (uint64_t i = threadIdx.x; i < hidden; i += blockDim.x) {
        const float d = xr[i] - mean;
        s2 = fmaf(d, d, s2);
    }
    const float var = block_sum(s2, sh) / (float)hidden;
    const float sd = sqrtf(var + eps);
    for (uint64_t i = threadIdx.x; i < hidden; i += blockDim.x) {
        float v = scale[i] * (xr[i] - mean) / sd;
        if (!RMS) v += bias[i];
        if (y) y[row * hidden + i] = v;
        if (y_xq) y_xq[xq_index(i, (uint32_t)row, bp)] = __float2half_rn(v);
        if (y_lp) y_lp[row * lp_ld + i] = f32_to_lp_bits(v, lp_bf16);
    }
}

// Many rows of up to 1024 elements: one wave per row (four rows per workgroup), the row read once
// in 16-byte pieces and kept in registers; no LDS, no barrier.  Same formulas as norm_token_kernel.
template <bool RMS, int U>
__global__ __launch_bounds__(256) void norm_rows_kernel(const float *__restrict__ x, uint64_t rows,
                                                        uint32_t hidden, const float *__restrict__ scale,
                                                        const float *__restrict__ bias, float eps, float *y,
                                                        __half *y_xq, uint32_t bp, uint16_t *y_lp,
                                                        uint64_t lp_ld, bool lp_bf16) {
    const uint32_t lane = threadIdx.x & 63;
    const uint64_t row = (uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float *xr = x + row * hidden;
    const uint32_t n4 = hidden / 4;
    float4 v[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const uint32_t i = lane + 64 * u;
        v[u] = i < n4 ? *(const float4 *)(xr + 4 * i) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    float mean = 0.f;
    if (!RMS) {
        float s = 0.f;
#pragma unroll
        for (int u = 0; u < U; u++) s += (v[u].x + v[u].y) + (v[u].z + v[u].w);
        mean = wave_sum(s) / (float)hidden;
    }
    float s2 = 0.f;
#pragma unroll
    for (int u = 0; u < U; u++) {
        if (lane + 64 * u < n4) {
            const float d0 = v[u].x - mean, d1 = v[u].y - mean, d2 = v[u].z - mean, d3 = v[u].w - mean;
            s2 = fmaf(d0, d0, s2); s2 = fmaf(d1, d1, s2); s2 = fmaf(d2, d2, s2); s2 = fmaf(d3, d3, s2);
        }
    }
    const float var = wave_sum(s2) / (float)hidden;
    const float rs = 1.0f / sqrtf(var + eps);
#pragma unroll
    for (int u = 0; u < U; u++) {
        const uint32_t i = lane + 64 * u;
        if (i >= n4) continue;
        const float4 sc = *(const float4 *)(scale + 4 * i);
        float o[4] = {sc.x * (v[u].x - mean) * rs, sc.y * (v[u].y - mean) * rs,
                      sc.z * (v[u].z - mean) * rs, sc.w * (v[u].w - mean) * rs};
        if (!RMS) {
            const float4 bi = *(const float4 *)(bias + 4 * i);
            o[0] += bi.x; o[1] += bi.y; o[2] += bi.z; o[3] += bi.w;
        }
        if (y) *(float4 *)(y + row * hidden + 4 * i) = make_float4(o[0], o[1], o[2], o[3]);
        if (y_xq) {
#pragma unroll
            for (int q = 0; q < 4; q++) y_xq[xq_index(4 * i + q, (uint32_t)row, bp)] = __float2half_rn(o[q]);
        }
        if (y_lp) {
            uint2 p;
            p.x = (uint32_t)f32_to_lp_bits(o[0], lp_bf16) | ((uint32_t)f32_to_lp_bits(o[1], lp_bf16) << 16);
            p.y = (uint32_t)f32_to_lp_bits(o[2], lp_bf16) | ((uint32_t)f32_to_lp_bits(o[3], lp_bf16) << 16);
            *(uint2 *)(y_lp + row * lp_ld + 4 * i) = p;
        }
    }
}

// Whole-slice statistics, single workgroup: exists for parity with the reference, and serves
// small slices and callers without a scratch buffer.  Sums are carried in f64 so the result is
// within an ulp or two of the reference's sequential Welford update.
template <bool RMS>
__global__ __launch_bounds__(1024) void norm_sequence_kernel(const float *__restrict__ x, uint64_t n,
                                                             uint64_t hidden,
                                                             const float *__restrict__ scale,
                                                             const float *__restrict__ bias,
                                                             float eps, float *y) {
    __shared__ double sh[16];
    double mean = 0.0;
    if (!RMS) {
        double s = 0.0;
        for (uint64_t i = threadIdx.x; i < n; i += blockDim.x) s += (double)x[i];
        mean = block_sum_f64(s, sh) / (double)n;
    }
    double s2 = 0.0;
    for (uint64_t i = threadIdx.x; i < n; i += blockDim.x) {
        const double d = (double)x[i] - mean;
        s2 += d * d;
    }
    const float var = (float)(block_sum_f64(s2, sh) / (double)n);
    const float sd = sqrtf(var + eps), meanf = (float)mean;
    for (uint64_t i = threadIdx.x; i < n; i += blockDim.x) {
        const uint64_t c = i % hidden;
        float v = scale[c] * (x[i] - meanf) / sd;
        if (!RMS) v += bias[c];
        y[i] = v;
    }
}

// The same over many workgroups, as two launches: partial sums, then apply.  Workgroup g owns
// elements [g * chunk, (g + 1) * chunk) and stores sum (x - c) and sum (x - c)^2 in f64, with c = x[0]
// (0 for RMSNorm): mean = c + S1 / n, variance = S2 / n - (S1 / n)^2.  Shifting by an element of the
// slice bounds the cancellation in that difference by n * 2^-53 relative to the variance (x[0] lies
// within sqrt(n) standard deviations of the mean), far below f32 rounding.  Every workgroup of the
// second launch adds up the partials in the same order, so all of them hold the same statistics.
// part: [2][kNormSeqMaxGroups] f64.
constexpr uint32_t kNormSeqMaxGroups = 256;
// PHASE 0: part[0][g], part[1][g].  PHASE 1: y.
template <bool RMS, int PHASE>
__global__ __launch_bounds__(256) void norm_sequence_part_kernel(const float *__restrict__ x, uint64_t n,
                                                                 uint64_t chunk, uint64_t hidden,
                                                                 const float *__restrict__ scale,
                                                                 const float *__restrict__ bias,
                                                                 float eps, double *part, float *y) {
    __shared__ double sh[16];
    const uint32_t G = gridDim.x, g = blockIdx.x;
    const uint64_t lo = (uint64_t)g * chunk, hi = lo + chunk < n ? lo + chunk : n;
    const double c = RMS ? 0.0 : (double)x[0];
    if (PHASE == 0) {
        double s1 = 0.0, s2 = 0.0;
        for (uint64_t i = lo + threadIdx.x; i < hi; i += blockDim.x) {
            const double d = (double)x[i] - c;
            s1 += d;
            s2 += d * d;
        }
        if (!RMS) s1 = block_sum_f64(s1, sh);
        s2 = block_sum_f64(s2, sh);
        if (threadIdx.x == 0) {
            part[g] = s1;
            part[kNormSeqMaxGroups + g] = s2;
        }
    } else {
        // (G <= 256 = blockDim.x: one partial per thread, summed in the same order by every workgroup)
        double s1 = !RMS && threadIdx.x < G ? part[threadIdx.x] : 0.0;
        double s2 = threadIdx.x < G ? part[kNormSeqMaxGroups + threadIdx.x] : 0.0;
        if (!RMS) s1 = block_sum_f64(s1, sh);
        s2 = block_sum_f64(s2, sh);
        const double mc = RMS ? 0.0 : s1 / (double)n;
        const float var = (float)(s2 / (double)n - mc * mc);
        const float sd = sqrtf(var + eps), meanf = (float)(c + mc);
        uint64_t col = (lo + threadIdx.x) % hidden;  // one division; then stepped along with i
        for (uint64_t i = lo + threadIdx.x; i < hi; i += blockDim.x) {
            float v = scale[col] * (x[i] - meanf) / sd;
            if (!RMS) v += bias[col];
            y[i] = v;
            col += blockDim.x;
            while (col >= hidden) col -= hidden;
        }
    }
}

size_t norm_sequence_scratch_bytes() { return 2 * kNormSeqMaxGroups * sizeof(double); }

int launch_norm(uint32_t kind, uint32_t scope, const float *x, uint64_t rows, uint64_t hidden,
                const float *scale, const float *bias, float eps, float *y, __half *y_xq,
                uint32_t bp, hipStream_t st, const LpOut *y_lp, double *partials) {
    if (rows == 0 || hidden == 0) return fail(COEUS_INVALID_INPUT, "empty normalisation input");
    uint16_t *lp = y_lp ? (uint16_t *)y_lp->p : nullptr;
    const uint64_t lp_ld = y_lp ? y_lp->ld : 0;
    const bool lp_bf = y_lp && y_lp->bf16;
    if (kind > 1 || scope > 1) return fail(COEUS_INVALID_INPUT, "unknown norm kind/scope");
    if (scope == COEUS_SCOPE_SEQUENCE) {
        if (y_xq || lp) return fail(COEUS_INVALID_INPUT, "whole-sequence norm has no 16-bit output");
        const uint64_t n = rows * hidden;
        if (partials && n >= 32768) {
            // at least 1024 elements per workgroup (128 x 768: 96 workgroups; with 4096 per workgroup
            // 24 CUs did the work of a launch that is all latency: 6.4 + 8.2 us)
            const uint32_t G = (uint32_t)std::min<uint64_t>(kNormSeqMaxGroups, n / 1024);
            const uint64_t chunk = ceil_div(n, G);
#define COEUS_NSP(RMSV, PH)                                                                          \
    hipLaunchKernelGGL((norm_sequence_part_kernel<RMSV, PH>), dim3(G), dim3(256), 0, st, x, n, chunk, \
                       hidden, scale, bias, eps, partials, y)
            if (kind == COEUS_NORM_RMSNORM) { COEUS_NSP(true, 0); COEUS_NSP(true, 1); }
            else { COEUS_NSP(false, 0); COEUS_NSP(false, 1); }
#undef COEUS_NSP
            COEUS_HIP(hipGetLastError());
            return COEUS_OK;
        }
        if (kind == COEUS_NORM_RMSNORM)
            hipLaunchKernelGGL(norm_sequence_kernel<true>, dim3(1), dim3(1024), 0, st, x, rows * hidden,
                               hidden, scale, bias, eps, y);
        else
            hipLaunchKernelGGL(norm_sequence_kernel<false>, dim3(1), dim3(1024), 0, st, x,
                               rows * hidden, hidden, scale, bias, eps, y);
    } else if (rows >= 512 && (hidden & 3) == 0 && hidden <= 1024 && (lp_ld & 3) == 0 && rows < (1ull << 33)) {
        // a prompt's worth of short rows: one wave per row (a workgroup per row leaves most of its lanes
        // idle there: 2.2 -> 4.5 TB/s at 768 elements; from 2048 elements up the workgroup per row is as
        // fast or faster, its four waves overlap one row's loads with another's arithmetic)
        const dim3 grid((unsigned)ceil_div(rows, 4));
        const bool rms = kind == COEUS_NORM_RMSNORM;
#define COEUS_NR(UV)                                                                                      \
    do {                                                                                                  \
        if (rms) hipLaunchKernelGGL((norm_rows_kernel<true, UV>), grid, dim3(256), 0, st, x, rows, (uint32_t)hidden, \
                                    scale, bias, eps, y, y_xq, bp, lp, lp_ld, lp_bf);                     \
        else hipLaunchKernelGGL((norm_rows_kernel<false, UV>), grid, dim3(256), 0, st, x, rows, (uint32_t)hidden,    \
                                scale, bias, eps, y, y_xq, bp, lp, lp_ld, lp_bf);                         \
    } while (0)
        if (hidden <= 256) COEUS_NR(1);
        else if (hidden <= 512) COEUS_NR(2);
        else COEUS_NR(4);
#undef COEUS_NR
    } else {
        if (kind == COEUS_NORM_RMSNORM)
            hipLaunchKernelGGL(norm_token_kernel<true>, dim3((unsigned)rows), dim3(256), 0, st, x, hidden,
                               scale, bias, eps, y, y_xq, bp, lp, lp_ld, lp_bf);
        else
            hipLaunchKernelGGL(norm_token_kernel<false>, dim3((unsigned)rows), dim3(256), 0, st, x,
                               hidden, scale, bias, eps, y, y_xq, bp, lp, lp_ld, lp_bf);
    }
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

// ids are range-checked on the host before upload (MT:816-822).  pos_dev (nullable) holds the
// position of row 0 on the device so a captured graph can be replayed as the context grows;
// with several sequences (rows == batch, one new token each) every row sits at that position.
template <bool BF16>
__global__ __launch_bounds__(1024) void embed_kernel(const void *__restrict__ table,
                                                     const float *__restrict__ pe,
                                                     const uint64_t *__restrict__ ids, uint64_t pos0,
                                                     const uint32_t *pos_dev, uint32_t rows_per_seq,
                                                     uint64_t hidden, float *x, float2 *stats,
                                                     const float *__restrict__ g_scale, float *g_out) {
    const uint64_t row = blockIdx.x;
    const uint64_t id = ids[row];
    const uint64_t pos = (pos_dev ? (uint64_t)*pos_dev : pos0) + row % rows_per_seq;
    const uint64_t stats_tiles = (hidden + 15) / 16;
    // 16 neighbouring lanes cover 16 consecutive elements: the loop bound is taken per group so
    // that a whole group runs the statistics shuffles together.  Four steps of the workgroup are
    // fetched before any is used: a decode step waits for this kernel's memory latency once.
    constexpr int U = 4;
    for (uint64_t g0 = threadIdx.x & ~15u; g0 < hidden; g0 += (uint64_t)U * blockDim.x) {
        float v[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const uint64_t i = g0 + (uint64_t)u * blockDim.x + (threadIdx.x & 15);
            v[u] = 0.f;
            if (i < hidden) {
                const float ev = BF16 ? bf16_bits_to_f32(((const uint16_t *)table)[id * hidden + i])
                                      : ((const float *)table)[id * hidden + i];
                v[u] = ev + pe[pos * hidden + i];
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const uint64_t i0 = g0 + (uint64_t)u * blockDim.x, i = i0 + (threadIdx.x & 15);
            if (i0 >= hidden) break;  // the same for the 16 lanes of a group
            const bool live = i < hidden;
            if (live) x[row * hidden + i] = v[u];
            if (live && g_out) g_out[row * hidden + i] = v[u] * g_scale[i];
            if (stats) {
                const uint64_t left = hidden - i0;
                const float2 r = group16_stats(v[u], live, left < 16 ? (uint32_t)left : 16u);
                if ((threadIdx.x & 15) == 0) stats[row * stats_tiles + i0 / 16] = r;
            }
        }
    }
}

int launch_embed(const void *table, bool table_bf16, const float *pe, const uint64_t *ids,
                 uint64_t rows, uint64_t rows_per_seq, uint64_t pos0, const uint32_t *pos_dev,
                 uint64_t hidden, float *x, float2 *stats, hipStream_t st, const float *g_scale, float *g_out) {
    if (rows == 0) return fail(COEUS_INVALID_INPUT, "empty embedding input");
    if (g_out && !g_scale) return fail(COEUS_INVALID_INPUT, "pre-scaled rows need the scale");
    // one lane per element up to 1024 (whole groups of 16); few rows (a decode step) are bound
    // by latency, many rows (a prompt) by the number of workgroups, which 256 lanes serve better
    const unsigned threads = rows > 64 ? 256u : (unsigned)std::min<uint64_t>(1024, round_up(hidden, 64));
    if (table_bf16)
        hipLaunchKernelGGL(embed_kernel<true>, dim3((unsigned)rows), dim3(threads), 0, st, table, pe, ids,
                           pos0, pos_dev, (uint32_t)rows_per_seq, hidden, x, stats, g_scale, g_out);
    else
        hipLaunchKernelGGL(embed_kernel<false>, dim3((unsigned)rows), dim3(threads), 0, st, table, pe, ids,
                           pos0, pos_dev, (uint32_t)rows_per_seq, hidden, x, stats, g_scale, g_out);
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

// The {sum, M2} record of every 16 consecutive elements of each row of h [rows, k]: what the
// producers of a decode step's residual stream write next to their outputs, as a launch of its own
// for callers that bring the rows from elsewhere.  One workgroup of 256 lanes per row.
__global__ __launch_bounds__(256) void row_stats16_kernel(const float *__restrict__ h, uint64_t k,
                                                          float2 *__restrict__ stats) {
    const uint64_t row = blockIdx.x, tiles = (k + 15) / 16;
    for (uint64_t i0 = threadIdx.x & ~15u; i0 < k; i0 += blockDim.x) {  // uniform per group of 16 lanes
        const uint64_t i = i0 + (threadIdx.x & 15);
        const bool live = i < k;
        const float v = live ? h[row * k + i] : 0.f;
        const uint64_t left = k - i0;
        const float2 r = group16_stats(v, live, left < 16 ? (uint32_t)left : 16u);
        if ((threadIdx.x & 15) == 0) stats[row * tiles + i0 / 16] = r;
    }
}

__global__ __launch_bounds__(256) void prescale_kernel(const float *__restrict__ h, const float *__restrict__ scale,
                                                       uint64_t k, float *__restrict__ g) {
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x, row = blockIdx.y;
    if (i < k) g[row * k + i] = h[row * k + i] * scale[i];
}

int launch_prescale(const float *h, const float *scale, uint64_t rows, uint64_t k, float *g, hipStream_t st) {
    if (rows == 0) return fail(COEUS_INVALID_INPUT, "pre-scaled rows: no rows");
    hipLaunchKernelGGL(prescale_kernel, dim3((unsigned)ceil_div(k, 256), (unsigned)rows), dim3(256), 0, st, h, scale, k, g);
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

int launch_row_stats16(const float *h, uint64_t rows, uint64_t k, float2 *stats, hipStream_t st) {
    if (rows == 0 || k == 0) return fail(COEUS_INVALID_INPUT, "empty statistics input");
    hipLaunchKernelGGL(row_stats16_kernel, dim3((unsigned)rows), dim3(256), 0, st, h, k, stats);
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

// argmax over each row of logits [rows, vocab]; lowest index wins ties.  One workgroup per row.
// With `advance` (pos, step; single-row launches only) the kernel also moves both counters on by
// one once its result is stored: the last act of a greedy decode step.
__global__ __launch_bounds__(1024) void argmax_kernel(const float *__restrict__ logits, uint64_t vocab,
                                                      uint64_t *out_ids, uint64_t *history,
                                                      uint64_t history_stride, const uint32_t *step_dev,
                                                      uint32_t *advance) {
    __shared__ float bv[16];
    __shared__ uint32_t bi[16];
    const uint64_t row = blockIdx.x;
    const float *l = logits + row * vocab;
    float best = -INFINITY;
    uint32_t idx = 0xffffffffu;
    auto take = [&](float v, uint32_t i) {
        if (v > best || (v == best && i < idx)) { best = v; idx = i; }
    };
    // 8 loads per lane are requested before the first comparison
    constexpr int U = 8;
    // 16-byte loads over the aligned middle of the row; up to 3 elements at either end one by one
    const uint32_t head = (uint32_t)((4 - ((row * vocab) & 3)) & 3);  // elements before the boundary
    const uint32_t hcut = head < vocab ? head : (uint32_t)vocab;
    const uint32_t n4 = (uint32_t)((vocab - hcut) / 4);
    const float4 *l4 = (const float4 *)(l + hcut);
    if (threadIdx.x < hcut) take(l[threadIdx.x], threadIdx.x);
    for (uint32_t base = threadIdx.x; base < n4; base += U * blockDim.x) {
        float4 v[U];
#pragma unroll
        for (int u = 0; u < U; u++) v[u] = l4[min(base + u * blockDim.x, n4 - 1)];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const uint32_t i = base + u * blockDim.x;  // ascending within a lane
            if (i < n4) {
                const uint32_t e0 = hcut + 4 * i;
                take(v[u].x, e0); take(v[u].y, e0 + 1); take(v[u].z, e0 + 2); take(v[u].w, e0 + 3);
            }
        }
    }
    {
        const uint32_t t0 = hcut + 4 * n4 + threadIdx.x;  // the last vocab - hcut - 4 n4 < 4 elements
        if (t0 < vocab) take(l[t0], t0);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(best, off, 64);
        const uint32_t oi = __shfl_xor(idx, off, 64);
        if (ov > best || (ov == best && oi < idx)) { best = ov; idx = oi; }
    }
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    if (lane == 0) { bv[wave] = best; bi[wave] = idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (uint32_t w = 1; w < nw; w++)
            if (bv[w] > best || (bv[w] == best && bi[w] < idx)) { best = bv[w]; idx = bi[w]; }
        if (idx == 0xffffffffu) idx = 0;  // all-NaN row
        out_ids[row] = idx;
        if (history) history[row * history_stride + (step_dev ? *step_dev : 0)] = idx;
        if (advance) { advance[0] += 1; advance[1] += 1; }
    }
}

int launch_argmax(const float *logits, uint64_t rows, uint64_t vocab, uint64_t *out_ids,
                  uint64_t *history, uint64_t history_stride, const uint32_t *step_dev,
                  hipStream_t st, uint32_t *advance) {
    if (advance && rows != 1)
        return fail(COEUS_INVALID_INPUT, "the position update rides on single-row argmax launches only");
    hipLaunchKernelGGL(argmax_kernel, dim3((unsigned)rows), dim3(1024), 0, st, logits, vocab, out_ids,
                       history, history_stride, step_dev, advance);
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

__global__ void advance_kernel(uint32_t *pos, uint32_t *step) {
    if (threadIdx.x == 0) { *pos += 1; *step += 1; }
}
int launch_advance(uint32_t *pos, uint32_t *step, hipStream_t st) {
    hipLaunchKernelGGL(advance_kernel, dim3(1), dim3(64), 0, st, pos, step);
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

}  // namespace coeus
