// Prefill matmul: C[m, n] = A[m, k] . W (math::matmul, MT:50-74) on the matrix cores.
//
//   gemm_f32_kernel   f32 weights [n][k]: v_mfma_f32_32x32x2_f32 (full f32 products and
//                     accumulation), 64x64 workgroup tile, 16-wide k slices staged in LDS.
//   gemm_lp_kernel    bf16 / Q8_0 / Q4_0 weights: v_mfma_f32_32x32x16_{bf16,f16}; activations are
//                     rounded to the matrix-core input type (bf16 for bf16 weights, f16 for
//                     quantised weights, whose integers and scales are exact in f16 products
//                     q*x with the block scale applied in f32).
#include "device_utils.hpp"

namespace coeus {

constexpr int BM = 64, BN = 64, BK = 16;

__global__ __launch_bounds__(256) void gemm_f32_kernel(const float *__restrict__ a,
                                                       const float *__restrict__ w, uint64_t m,
                                                       uint64_t n, uint64_t k, EpiArgs e) {
    // k-major tiles: element (row, kk) at [kk][row]; +4 padding keeps the transposing stores
    // and the 32-consecutive-row MFMA operand reads off the same banks
    __shared__ float as[BK][BM + 4];
    __shared__ float ws[BK][BN + 4];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint64_t m0 = (uint64_t)blockIdx.y * BM, n0 = (uint64_t)blockIdx.x * BN;
    const uint32_t wm = (wave >> 1) * 32, wn = (wave & 1) * 32;
    float16_t acc;
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = 0.f;

    const uint32_t lrow = tid >> 2, lk = (tid & 3) * 4;  // 64 rows x 4 float4 per tile
    const bool vec = (k & 3) == 0;
    for (uint64_t k0 = 0; k0 < k; k0 += BK) {
        float av[4] = {0.f, 0.f, 0.f, 0.f}, wv[4] = {0.f, 0.f, 0.f, 0.f};
        const uint64_t ar = m0 + lrow, wr = n0 + lrow, kk = k0 + lk;
        if (vec && kk + 4 <= k) {
            if (ar < m) { const float4 t = *(const float4 *)(a + ar * k + kk); av[0] = t.x; av[1] = t.y; av[2] = t.z; av[3] = t.w; }
            if (wr < n) { const float4 t = *(const float4 *)(w + wr * k + kk); wv[0] = t.x; wv[1] = t.y; wv[2] = t.z; wv[3] = t.w; }
        } else {
#pragma unroll
            for (int t = 0; t < 4; t++) {
                if (ar < m && kk + t < k) av[t] = a[ar * k + kk + t];
                if (wr < n && kk + t < k) wv[t] = w[wr * k + kk + t];
            }
        }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < 4; t++) {
            as[lk + t][lrow] = av[t];
            ws[lk + t][lrow] = wv[t];
        }
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < BK; ks += 2) {
            const float fa = as[ks + (lane >> 5)][wm + (lane & 31)];
            const float fb = ws[ks + (lane >> 5)][wn + (lane & 31)];
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa, fb, acc, 0, 0, 0);
        }
    }
    // accumulator i of lane l: row 8*(i/4) + 4*(l/32) + i%4, column l%32
    const uint64_t col = n0 + wn + (lane & 31);
    const bool gated = e.act == COEUS_EPI_SILU_GATE;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const uint64_t row = m0 + wm + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
        // gated: columns (2c, 2c+1) hold (gate_c, up_c) and sit in neighbouring lanes
        const float other = __shfl_xor(acc[i], 1, 64);
        if (row >= m || col >= n) continue;
        if (!gated) epi_store(e, row, col, acc[i]);
        else if ((lane & 1) == 0) epi_store_gated(e, row, col >> 1, acc[i], other);
    }
}

static int launch_gemm_f32(const Weight &w, const float *a, uint64_t m, const Epilogue &ep, hipStream_t st) {
    const EpiArgs e = make_epi(ep, w.n);
    const dim3 grid((unsigned)ceil_div(w.n, BN), (unsigned)ceil_div(m, BM));
    hipLaunchKernelGGL(gemm_f32_kernel, grid, dim3(256), 0, st, a, (const float *)w.data, m, w.n, w.k, e);
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

// ---------------------------------------------------------------- 16-bit inputs
// C = A . W^T with A [m][k] and W [n][k] both 16-bit row-major (k contiguous): every lane feeds
// the matrix core 8 consecutive k of one row, for both operands.
constexpr int HM = 128, HN = 128, HK = 32, HLD = 40;  // LDS row stride in elements (80 B)

template <bool BF16>
__global__ __launch_bounds__(256) void gemm_h_kernel(const uint16_t *__restrict__ a,
                                                     const uint16_t *__restrict__ w, uint64_t m,
                                                     uint64_t n, uint64_t k, EpiArgs e) {
    __shared__ __attribute__((aligned(16))) uint16_t as[HM * HLD];
    __shared__ __attribute__((aligned(16))) uint16_t ws[HN * HLD];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint64_t m0 = (uint64_t)blockIdx.y * HM, n0 = (uint64_t)blockIdx.x * HN;
    const uint32_t wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
    float16_t acc[2][2];
#pragma unroll
    for (int x = 0; x < 2; x++)
#pragma unroll
        for (int y = 0; y < 2; y++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[x][y][i] = 0.f;

    const uint32_t lrow = tid >> 1, lseg = (tid & 1) * 16;
    const bool vec = (k & 7) == 0;
    auto load16 = [&](const uint16_t *base, uint64_t row, uint64_t rows, uint64_t kk, uint4 &lo, uint4 &hi) {
        lo = make_uint4(0, 0, 0, 0);
        hi = make_uint4(0, 0, 0, 0);
        if (row >= rows) return;
        const uint16_t *p = base + row * k + kk;
        if (vec) {
            if (kk + 8 <= k) lo = *(const uint4 *)p;
            if (kk + 16 <= k) hi = *(const uint4 *)(p + 8);
        } else {
            uint16_t t[16];
#pragma unroll
            for (int u = 0; u < 16; u++) t[u] = kk + u < k ? p[u] : (uint16_t)0;
            lo = make_uint4(t[0] | (uint32_t)t[1] << 16, t[2] | (uint32_t)t[3] << 16, t[4] | (uint32_t)t[5] << 16, t[6] | (uint32_t)t[7] << 16);
            hi = make_uint4(t[8] | (uint32_t)t[9] << 16, t[10] | (uint32_t)t[11] << 16, t[12] | (uint32_t)t[13] << 16, t[14] | (uint32_t)t[15] << 16);
        }
    };
    uint4 alo, ahi, wlo, whi;
    load16(a, m0 + lrow, m, lseg, alo, ahi);
    load16(w, n0 + lrow, n, lseg, wlo, whi);
    for (uint64_t k0 = 0; k0 < k; k0 += HK) {
        __syncthreads();
        *(uint4 *)(as + lrow * HLD + lseg) = alo;
        *(uint4 *)(as + lrow * HLD + lseg + 8) = ahi;
        *(uint4 *)(ws + lrow * HLD + lseg) = wlo;
        *(uint4 *)(ws + lrow * HLD + lseg + 8) = whi;
        __syncthreads();
        if (k0 + HK < k) {  // prefetch the next slice while the matrix cores work on this one
            load16(a, m0 + lrow, m, k0 + HK + lseg, alo, ahi);
            load16(w, n0 + lrow, n, k0 + HK + lseg, wlo, whi);
        }
#pragma unroll
        for (int ks = 0; ks < HK; ks += 16) {
            uint4 af[2], bf[2];
#pragma unroll
            for (int x = 0; x < 2; x++) {
                af[x] = *(const uint4 *)(as + (wm + x * 32 + (lane & 31)) * HLD + ks + 8 * (lane >> 5));
                bf[x] = *(const uint4 *)(ws + (wn + x * 32 + (lane & 31)) * HLD + ks + 8 * (lane >> 5));
            }
#pragma unroll
            for (int x = 0; x < 2; x++)
#pragma unroll
                for (int y = 0; y < 2; y++) {
                    if (BF16) {
                        union { uint4 u; bf16x8_t v; } ua, ub;
                        ua.u = af[x]; ub.u = bf[y];
                        acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ua.v, ub.v, acc[x][y], 0, 0, 0);
                    } else {
                        union { uint4 u; half8_t v; } ua, ub;
                        ua.u = af[x]; ub.u = bf[y];
                        acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ua.v, ub.v, acc[x][y], 0, 0, 0);
                    }
                }
        }
    }
    const bool gated = e.act == COEUS_EPI_SILU_GATE;
#pragma unroll
    for (int x = 0; x < 2; x++)
#pragma unroll
        for (int y = 0; y < 2; y++) {
            const uint64_t col = n0 + wn + y * 32 + (lane & 31);
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const uint64_t row = m0 + wm + x * 32 + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
                const float other = __shfl_xor(acc[x][y][i], 1, 64);
                if (row >= m || col >= n) continue;
                if (!gated) epi_store(e, row, col, acc[x][y][i]);
                else if ((lane & 1) == 0) epi_store_gated(e, row, col >> 1, acc[x][y][i], other);
            }
        }
}

int launch_gemm(const Weight &w, const float *a, uint64_t m, const Epilogue &ep, GemmScratch &scr,
                hipStream_t st) {
    if (m == 0) return fail(COEUS_INVALID_INPUT, "matmul with zero rows");
    if (ep.act == COEUS_EPI_SILU_GATE && (w.n & 1))
        return fail(COEUS_INVALID_INPUT, "gated epilogue needs an even number of weight rows");
    if (ep.out_xq) return fail(COEUS_INVALID_INPUT, "prefill matmul has no xq output");
    if (w.dtype == COEUS_W_F32) return launch_gemm_f32(w, a, m, ep, st);
    const uint64_t a_bytes = m * w.k * 2;
    if (!scr.a_lp || scr.a_lp_bytes < a_bytes)
        return fail(COEUS_INVALID_INPUT, "matmul staging buffer too small (%llu < %llu bytes)",
                    (unsigned long long)scr.a_lp_bytes, (unsigned long long)a_bytes);
    const uint16_t *wp = (const uint16_t *)w.data;
    const bool bf = w.dtype == COEUS_W_BF16;
    if (bf) {
        COEUS_TRY(launch_f32_to_bf16(a, (uint16_t *)scr.a_lp, m * w.k, st));
    } else {
        const uint64_t w_bytes = w.n * w.k * 2;
        if (!scr.w_lp || scr.w_lp_bytes < w_bytes)
            return fail(COEUS_INVALID_INPUT, "weight staging buffer too small (%llu < %llu bytes)",
                        (unsigned long long)scr.w_lp_bytes, (unsigned long long)w_bytes);
        COEUS_TRY(launch_f32_to_f16(a, (__half *)scr.a_lp, m * w.k, st));
        COEUS_TRY(launch_dequant_to_f16(w, (__half *)scr.w_lp, st));
        wp = (const uint16_t *)scr.w_lp;
    }
    const EpiArgs e = make_epi(ep, w.n);
    const dim3 grid((unsigned)ceil_div(w.n, HN), (unsigned)ceil_div(m, HM));
    if (bf)
        hipLaunchKernelGGL(gemm_h_kernel<true>, grid, dim3(256), 0, st, (const uint16_t *)scr.a_lp, wp, m, w.n, w.k, e);
    else
        hipLaunchKernelGGL(gemm_h_kernel<false>, grid, dim3(256), 0, st, (const uint16_t *)scr.a_lp, wp, m, w.n, w.k, e);
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

}  // namespace coeus
