// Prefill matmul: C[m, n] = A[m, k] . W (math::matmul, MT:50-74) on the matrix cores.
//
//   gemm_f32_kernel   f32 weights [n][k]: v_mfma_f32_32x32x2_f32 (full f32 products and
//                     accumulation), 64x64 workgroup tile, 32-wide k slices staged in LDS, three
//                     slices requested ahead.
//   16-bit kernels    bf16 / Q8_0 / Q4_0 weights: v_mfma_f32_32x32x16_{bf16,f16}; activations are
//                     rounded to the matrix-core input type (bf16 for bf16 weights, f16 for
//                     quantised weights, which are expanded to f16(q * d) first).
//     gemm_h256k64_kernel  k % 64 == 0: 256x256 tile, four waves of 128x128, 64-wide k slices
//                          loaded straight into a ring of five LDS regions
//     gemm_h256_kernel     k % 32 == 0: 256x256 tile, eight waves of 128x64, 32-wide slices
//     gemm_h_kernel        any k: 128x128 tile, register-staged
//     gemm_qskinny_kernel  up to 64 rows on quantised weights: streams the quantised blocks
//     gemm_split_reduce_kernel, gemm_tail_reduce_kernel: sums behind launches split along k
#include "device_utils.hpp"

namespace coeus {

constexpr int BM = 64, BN = 64, BK = 32, F32_AHEAD = 3;

// One k slice of both operands for this thread: 2 + 2 pieces of 4 consecutive k (64 rows x 32 k per
// operand = 512 pieces over 256 threads), zero past the edges.
struct F32Slice { float4 a0, a1, w0, w1; };

// VEC (k % 4 == 0): one unconditional 16-byte load from a clamped address, zeroed afterwards if the
// piece lies outside the matrix.  (A load under a branch would make the compiler wait for every
// load in flight, the slices requested ahead included, before the first use.)
template <bool VEC>
__device__ __forceinline__ float4 f32_piece(const float *__restrict__ base, uint64_t row, uint64_t rows,
                                            uint64_t k, uint64_t kk) {
    if (VEC) {
        const bool in = row < rows && kk < k;  // k % 4 == 0: a piece is all in or all out
        const float4 t = *(const float4 *)(base + (row < rows ? row : rows - 1) * k + (kk < k ? kk : 0));
        return in ? t : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (row >= rows) return v;
    if (kk < k) v.x = base[row * k + kk];
    if (kk + 1 < k) v.y = base[row * k + kk + 1];
    if (kk + 2 < k) v.z = base[row * k + kk + 2];
    if (kk + 3 < k) v.w = base[row * k + kk + 3];
    return v;
}

template <bool VEC>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const float *__restrict__ a,
                                                       const float *__restrict__ w, uint64_t m,
                                                       uint64_t n, uint64_t k, EpiArgs e) {
    // k-major tiles: element (row, kk) at [kk][row]; +4 padding keeps the transposing stores
    // and the 32-consecutive-row MFMA operand reads off the same banks.  Two buffers: a slice is
    // written while the previous one is multiplied, one barrier per slice.
    __shared__ float as[2][BK][BM + 4];
    __shared__ float ws[2][BK][BN + 4];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint64_t m0 = (uint64_t)blockIdx.y * BM, n0 = (uint64_t)blockIdx.x * BN;
    const uint32_t wm = (wave >> 1) * 32, wn = (wave & 1) * 32;
    float16_t acc;
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = 0.f;

    // piece p = tid + 256 u (u = 0, 1): row p / 8, k offset 4 (p % 8)
    const uint32_t lrow = tid >> 3, lk = (tid & 7) * 4;
    const uint64_t nslices = (k + BK - 1) / BK;
    auto fetch = [&](uint64_t sl) -> F32Slice {
        F32Slice f;
        const uint64_t kk = sl * BK + lk;
        f.a0 = f32_piece<VEC>(a, m0 + lrow, m, k, kk);
        f.a1 = f32_piece<VEC>(a, m0 + lrow + 32, m, k, kk);
        f.w0 = f32_piece<VEC>(w, n0 + lrow, n, k, kk);
        f.w1 = f32_piece<VEC>(w, n0 + lrow + 32, n, k, kk);
        return f;
    };
    auto put = [&](uint32_t buf, const F32Slice &f) {
        as[buf][lk][lrow] = f.a0.x; as[buf][lk + 1][lrow] = f.a0.y; as[buf][lk + 2][lrow] = f.a0.z; as[buf][lk + 3][lrow] = f.a0.w;
        as[buf][lk][lrow + 32] = f.a1.x; as[buf][lk + 1][lrow + 32] = f.a1.y; as[buf][lk + 2][lrow + 32] = f.a1.z; as[buf][lk + 3][lrow + 32] = f.a1.w;
        ws[buf][lk][lrow] = f.w0.x; ws[buf][lk + 1][lrow] = f.w0.y; ws[buf][lk + 2][lrow] = f.w0.z; ws[buf][lk + 3][lrow] = f.w0.w;
        ws[buf][lk][lrow + 32] = f.w1.x; ws[buf][lk + 1][lrow + 32] = f.w1.y; ws[buf][lk + 2][lrow + 32] = f.w1.z; ws[buf][lk + 3][lrow + 32] = f.w1.w;
    };
    auto mult = [&](uint32_t buf) {
#pragma unroll
        for (int ks = 0; ks < BK; ks += 2) {
            const float fa = as[buf][ks + (lane >> 5)][wm + (lane & 31)];
            const float fb = ws[buf][ks + (lane >> 5)][wn + (lane & 31)];
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa, fb, acc, 0, 0, 0);
        }
    };
    // Three slices travel from memory while one is multiplied (small problems are a chain of
    // slices per workgroup: what bounds them is the memory latency per slice, not the bandwidth).
    // Slices past the end come back as zeros.
    F32Slice f0 = fetch(0), f1 = fetch(1), f2 = fetch(2);
    for (uint64_t sl = 0; sl < nslices; sl += F32_AHEAD) {
        put((uint32_t)(sl & 1), f0);
        __syncthreads();
        f0 = fetch(sl + 3);
        mult((uint32_t)(sl & 1));
        if (sl + 1 >= nslices) break;
        put((uint32_t)((sl + 1) & 1), f1);
        __syncthreads();
        f1 = fetch(sl + 4);
        mult((uint32_t)((sl + 1) & 1));
        if (sl + 2 >= nslices) break;
        put((uint32_t)((sl + 2) & 1), f2);
        __syncthreads();
        f2 = fetch(sl + 5);
        mult((uint32_t)((sl + 2) & 1));
    }
    // accumulator i of lane l: row 8*(i/4) + 4*(l/32) + i%4, column l%32
    const uint64_t col = n0 + wn + (lane & 31);
    const bool gated = e.act == COEUS_EPI_SILU_GATE;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const uint64_t row = m0 + wm + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
        // gated: columns (2c, 2c+1) hold (gate_c, up_c) and sit in neighbouring lanes
        const float other = lane_xor1(acc[i]);
        if (row >= m || col >= n) continue;
        if (!gated) epi_store(e, row, col, acc[i]);
        else if ((lane & 1) == 0) epi_store_gated(e, row, col >> 1, acc[i], other);
    }
}

// The same product for outputs too small to give every CU a 64x64 tile (a prompt of 128 tokens
// has 2 x 12 of them for a 768-wide projection): 32x32 tiles, and the workgroup's four waves split
// every k slice between them (wave v takes k 8v..8v+7 of each 32), so a workgroup's chain of
// slices costs a quarter of the matrix-core time per slice.  A wave fetches and stages exactly the
// 32 x 8 pieces of both operands that it multiplies, in its own part of LDS: no wave waits for
// another inside the loop (LDS serves a wave's stores and loads in order, so there is no barrier
// at all), and each runs six slices of its own requests ahead.  The four partial tiles are added
// through LDS at the end (a different summation order from the 64x64 kernel, the same products).
constexpr int SM = 32, SN = 32, F32S_AHEAD = 6;
struct F32SliceS { float4 a, w; };

template <bool VEC>
__global__ __launch_bounds__(256) void gemm_f32_small_kernel(const float *__restrict__ a,
                                                             const float *__restrict__ w, uint64_t m,
                                                             uint64_t n, uint64_t k, uint32_t splits, EpiArgs e) {
    __shared__ float as[4][2][8][SM + 4];  // per wave: two buffers of 8 k x 32 rows, k-major
    __shared__ float ws[4][2][8][SN + 4];
    __shared__ float red[4][16][64];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint64_t m0 = (uint64_t)blockIdx.y * SM, n0 = (uint64_t)blockIdx.x * SN;
    float16_t acc;
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = 0.f;
    const uint32_t lrow = lane >> 1, lk = (lane & 1) * 4;  // the wave's 32 rows x 2 pieces per operand and slice
    // blockIdx.z: this workgroup's share of the slices (a launch split along k stores bare products
    // into plane blockIdx.z of e.out_f32, gemm_split_reduce_kernel sums the planes)
    const uint64_t all_slices = (k + BK - 1) / BK;
    const uint64_t sbeg = all_slices * blockIdx.z / splits, nslices = all_slices * (blockIdx.z + 1) / splits;
    if (splits > 1) e.out_f32 += (uint64_t)blockIdx.z * m * e.n_eff;
    auto fetch = [&](uint64_t sl) -> F32SliceS {
        F32SliceS f;
        f.a = f32_piece<VEC>(a, m0 + lrow, m, k, sl * BK + 8 * wave + lk);
        f.w = f32_piece<VEC>(w, n0 + lrow, n, k, sl * BK + 8 * wave + lk);
        return f;
    };
    auto put = [&](uint32_t buf, const F32SliceS &f) {
        float(*pa)[SM + 4] = as[wave][buf];
        float(*pw)[SN + 4] = ws[wave][buf];
        pa[lk][lrow] = f.a.x; pa[lk + 1][lrow] = f.a.y; pa[lk + 2][lrow] = f.a.z; pa[lk + 3][lrow] = f.a.w;
        pw[lk][lrow] = f.w.x; pw[lk + 1][lrow] = f.w.y; pw[lk + 2][lrow] = f.w.z; pw[lk + 3][lrow] = f.w.w;
    };
    auto mult = [&](uint32_t buf) {
#pragma unroll
        for (int ks = 0; ks < 8; ks += 2) {
            const float fa = as[wave][buf][ks + (lane >> 5)][lane & 31];
            const float fb = ws[wave][buf][ks + (lane >> 5)][lane & 31];
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa, fb, acc, 0, 0, 0);
        }
    };
    F32SliceS f0 = fetch(sbeg), f1 = fetch(sbeg + 1), f2 = fetch(sbeg + 2), f3 = fetch(sbeg + 3), f4 = fetch(sbeg + 4),
              f5 = fetch(sbeg + 5);
    // (reading a slice's fragments one step ahead of their products, in a register double buffer,
    // changed nothing: a launch is 2 us of launch, 2-3 us until the first operands arrive, 0.14 us per
    // slice of four chained matrix instructions and 1.5 us of epilogue)
#define COEUS_F32S_STEP(F, OFF)                                    \
    if (sl + OFF >= nslices) break;                                \
    put((uint32_t)((sl + OFF) & 1), F);                            \
    F = fetch(sl + OFF + F32S_AHEAD);                              \
    mult((uint32_t)((sl + OFF) & 1));
    for (uint64_t sl = sbeg; sl < nslices; sl += F32S_AHEAD) {
        COEUS_F32S_STEP(f0, 0)
        COEUS_F32S_STEP(f1, 1)
        COEUS_F32S_STEP(f2, 2)
        COEUS_F32S_STEP(f3, 3)
        COEUS_F32S_STEP(f4, 4)
        COEUS_F32S_STEP(f5, 5)
    }
#undef COEUS_F32S_STEP
#pragma unroll
    for (int i = 0; i < 16; i++) red[wave][i][lane] = acc[i];
    __syncthreads();
    // wave v finishes accumulator elements 4v..4v+3: rows 8v + 4 (l / 32) + 0..3, column l % 32
    const uint64_t col = n0 + (lane & 31);
    const bool gated = e.act == COEUS_EPI_SILU_GATE;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int i = 4 * wave + q;
        const float v = (red[0][i][lane] + red[1][i][lane]) + (red[2][i][lane] + red[3][i][lane]);
        const uint64_t row = m0 + 8 * wave + 4 * (lane >> 5) + q;
        const float other = lane_xor1(v);
        if (row >= m || col >= n) continue;
        if (!gated) epi_store(e, row, col, v);
        else if ((lane & 1) == 0) epi_store_gated(e, row, col >> 1, v, other);
    }
}

__global__ void gemm_split_reduce_kernel(const float *__restrict__ part, uint32_t splits, uint64_t m, uint64_t n,
                                         EpiArgs e);  // (defined with the 16-bit kernels below)

static bool gemm_f32_is_small(const Weight &w, uint64_t m) {
    return ceil_div(w.n, BN) * ceil_div(m, BM) < 256;  // fewer 64x64 tiles than CUs
}

// The 32x32-tile kernel takes 7-8 us plus about 0.3 us per 32-wide slice of k whatever the launch's
// size, so a long k on few tiles (the FFN's second matmul on a 128-token prompt: 96 slices, 96
// workgroups, 36-41 us) is split along k over up to 8 workgroups per tile, at least 12 slices each
// and about three workgroups per CU in all, and gemm_split_reduce_kernel sums the planes in split
// order and runs the epilogue (8 + 5 us).  Below 48 slices the second launch costs what the split
// saves (768-long k, 128 rows: 16.5 us unsplit, 17.7 + 4.7 us in two shares).
static uint32_t gemm_f32_splits_wanted(const Weight &w, uint64_t m) {
    if (w.dtype != COEUS_W_F32 || m == 0 || !gemm_f32_is_small(w, m)) return 1;
    const uint64_t wgs = ceil_div(w.n, SN) * ceil_div(m, SM), slices = ceil_div(w.k, BK);
    if (slices < 48) return 1;
    uint64_t s = 768 / wgs;
    if (s > slices / 12) s = slices / 12;
    if (s > 8) s = 8;
    return s < 2 ? 1 : (uint32_t)s;
}

static int launch_gemm_f32(const Weight &w, const float *a, uint64_t m, const Epilogue &ep,
                           const GemmScratch &scr, hipStream_t st) {
    const EpiArgs e = make_epi(ep, w.n);
    const dim3 grid((unsigned)ceil_div(w.n, BN), (unsigned)ceil_div(m, BM));
    const bool small = gemm_f32_is_small(w, m);
    uint32_t splits = gemm_f32_splits_wanted(w, m);
    if (splits > 1 && (!scr.partials || scr.partials_bytes < (uint64_t)splits * m * w.n * 4)) splits = 1;
    const dim3 sgrid((unsigned)ceil_div(w.n, SN), (unsigned)ceil_div(m, SM), splits);
    EpiArgs plain;  // a split launch stores bare products: [split][m][n] f32
    if (splits > 1) {
        Epilogue pe;
        pe.out_f32 = scr.partials;
        plain = make_epi(pe, w.n);
    }
    const EpiArgs &ke = splits > 1 ? plain : e;
    const uint64_t groups = ceil_div(w.n, e.act == COEUS_EPI_SILU_GATE ? 8 : 4);
    if (scr.ev_begin) COEUS_HIP(hipEventRecord(scr.ev_begin, st));
    for (uint32_t rep = 0; rep < (scr.repeat ? scr.repeat : 1); rep++) {
        if (small && (w.k & 3) == 0)
            hipLaunchKernelGGL(gemm_f32_small_kernel<true>, sgrid, dim3(256), 0, st, a, (const float *)w.data, m, w.n, w.k, splits, ke);
        else if (small)
            hipLaunchKernelGGL(gemm_f32_small_kernel<false>, sgrid, dim3(256), 0, st, a, (const float *)w.data, m, w.n, w.k, splits, ke);
        else if ((w.k & 3) == 0)
            hipLaunchKernelGGL(gemm_f32_kernel<true>, grid, dim3(256), 0, st, a, (const float *)w.data, m, w.n, w.k, e);
        else
            hipLaunchKernelGGL(gemm_f32_kernel<false>, grid, dim3(256), 0, st, a, (const float *)w.data, m, w.n, w.k, e);
        if (splits > 1)
            hipLaunchKernelGGL(gemm_split_reduce_kernel, dim3((unsigned)ceil_div(m * groups, 256)), dim3(256), 0, st,
                               (const float *)scr.partials, splits, m, w.n, e);
    }
    if (scr.ev_end) COEUS_HIP(hipEventRecord(scr.ev_end, st));
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
                                                     uint64_t n, uint64_t k, uint64_t lda,
                                                     uint64_t ldw, EpiArgs e) {
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
    const bool vec = ((k | lda | ldw) & 7) == 0;
    auto load16 = [&](const uint16_t *base, uint64_t ld, uint64_t row, uint64_t rows, uint64_t kk, uint4 &lo, uint4 &hi) {
        lo = make_uint4(0, 0, 0, 0);
        hi = make_uint4(0, 0, 0, 0);
        if (row >= rows) return;
        const uint16_t *p = base + row * ld + kk;
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
    load16(a, lda, m0 + lrow, m, lseg, alo, ahi);
    load16(w, ldw, n0 + lrow, n, lseg, wlo, whi);
    for (uint64_t k0 = 0; k0 < k; k0 += HK) {
        __syncthreads();
        *(uint4 *)(as + lrow * HLD + lseg) = alo;
        *(uint4 *)(as + lrow * HLD + lseg + 8) = ahi;
        *(uint4 *)(ws + lrow * HLD + lseg) = wlo;
        *(uint4 *)(ws + lrow * HLD + lseg + 8) = whi;
        __syncthreads();
        if (k0 + HK < k) {  // prefetch the next slice while the matrix cores work on this one
            load16(a, lda, m0 + lrow, m, k0 + HK + lseg, alo, ahi);
            load16(w, ldw, n0 + lrow, n, k0 + HK + lseg, wlo, whi);
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
                const float other = lane_xor1(acc[x][y][i]);
                if (row >= m || col >= n) continue;
                if (!gated) epi_store(e, row, col, acc[x][y][i]);
                else if ((lane & 1) == 0) epi_store_gated(e, row, col >> 1, acc[x][y][i], other);
            }
        }
}

// ---------------------------------------------------------------- epilogue of the 16-bit matmuls
// Shared by the matmul kernel (accumulators laid out row-major through an LDS strip) and by the
// kernel that sums the partial products of a k-split launch.

// Where 4 consecutive output columns starting at `col` of a prompt pass's q|k|v projection go:
// the key and value thirds are written into the cache (4 consecutive dims of one head).
struct KvCols {
    bool on;
    char *dst;
    uint64_t off;
};
__device__ __forceinline__ KvCols epi_kv_cols(const EpiArgs &e, uint64_t col, uint64_t n) {
    KvCols kc{false, nullptr, 0};
    kc.on = e.kv_k && e.kv_rows_per_seq && col >= e.kv_inner && col + 3 < n;
    if (kc.on) {
        const uint32_t cc = (uint32_t)col;
        const bool is_k = cc < 2 * e.kv_inner;
        const uint32_t c = cc - (is_k ? 1u : 2u) * e.kv_inner, hh = c / e.kv_hd, d = c % e.kv_hd;
        kc.dst = (char *)(is_k ? e.kv_k : e.kv_v);
        kc.off = (uint64_t)hh * e.kv_max_ctx * e.kv_hd + d;
    }
    return kc;
}
__device__ __forceinline__ void epi_store4(const EpiArgs &e, uint64_t row, uint64_t col, const float (&v)[4]) {
    if (e.out_f32) *(float4 *)(e.out_f32 + row * e.n_eff + col) = make_float4(v[0], v[1], v[2], v[3]);
    if (e.out_lp) {
        uint2 p;
        p.x = (uint32_t)f32_to_lp_bits(v[0], e.lp_bf16) | ((uint32_t)f32_to_lp_bits(v[1], e.lp_bf16) << 16);
        p.y = (uint32_t)f32_to_lp_bits(v[2], e.lp_bf16) | ((uint32_t)f32_to_lp_bits(v[3], e.lp_bf16) << 16);
        *(uint2 *)(e.out_lp + row * e.lp_ld + col) = p;
    }
}
__device__ __forceinline__ bool epi_vec4(const EpiArgs &e) {
    return (e.n_eff & 3) == 0 && (e.lp_ld & 3) == 0 && (e.out_f32 || e.out_lp) && !e.out_xq;
}
// Columns col .. col + 3 of activation row `row` (bias, cache append or activation, residual, store).
__device__ __forceinline__ void epi_row4(const EpiArgs &e, bool vec4, const KvCols &kc, uint64_t row,
                                         uint64_t col, uint64_t n, float (&v)[4]) {
    if (vec4 && col + 3 < n) {
        if (e.bias) {
            const float4 b4 = *(const float4 *)(e.bias + col);
            v[0] += b4.x; v[1] += b4.y; v[2] += b4.z; v[3] += b4.w;
        }
        if (kc.on) {
            const uint32_t sq = (uint32_t)row / e.kv_rows_per_seq, tok = (uint32_t)row - sq * e.kv_rows_per_seq;
            const uint64_t idx = ((uint64_t)sq * e.kv_heads * e.kv_max_ctx + e.kv_pos0 + tok) * e.kv_hd + kc.off;
            if (e.kv_dtype == COEUS_KV_F32) {
                *(float4 *)((float *)kc.dst + idx) = make_float4(v[0], v[1], v[2], v[3]);
            } else {
                const bool kbf = e.kv_dtype == COEUS_KV_BF16;
                uint2 p;
                p.x = (uint32_t)f32_to_lp_bits(v[0], kbf) | ((uint32_t)f32_to_lp_bits(v[1], kbf) << 16);
                p.y = (uint32_t)f32_to_lp_bits(v[2], kbf) | ((uint32_t)f32_to_lp_bits(v[3], kbf) << 16);
                *(uint2 *)((uint16_t *)kc.dst + idx) = p;
            }
            return;
        }
        if (e.act == COEUS_EPI_GELU)
#pragma unroll
            for (int q = 0; q < 4; q++) v[q] = gelu_tanh(v[q]);
        if (e.residual) {
            const float4 r4 = *(const float4 *)(e.residual + row * e.n_eff + col);
            v[0] += r4.x; v[1] += r4.y; v[2] += r4.z; v[3] += r4.w;
        }
        epi_store4(e, row, col, v);
    } else {
#pragma unroll
        for (int q = 0; q < 4; q++)
            if (col + q < n) epi_store(e, row, col + q, v[q]);
    }
}
// Gated outputs ocol .. ocol + 3 of row `row`, from the weight rows (gate, up) = raw columns
// raw .. raw + 7 (raw = 2 ocol).
__device__ __forceinline__ void epi_row4_gated(const EpiArgs &e, bool vec4, uint64_t row, uint64_t ocol,
                                               uint64_t raw, uint64_t n, const float (&gv)[4],
                                               const float (&uv)[4]) {
    if (vec4 && !e.bias && !e.residual && raw + 7 < n) {
        float o[4];
#pragma unroll
        for (int q = 0; q < 4; q++) o[q] = silu(gv[q]) * uv[q];
        epi_store4(e, row, ocol, o);
    } else {
#pragma unroll
        for (int q = 0; q < 4; q++)
            if (raw + 2 * q + 1 < n) epi_store_gated(e, row, ocol + q, gv[q], uv[q]);
    }
}

// Sums the partial products of a k-split launch ([splits][m][n] f32, split s holding the products
// over its share of k) in split order and runs the epilogue.  One thread per 4 outputs of a row.
__global__ __launch_bounds__(256) void gemm_split_reduce_kernel(const float *__restrict__ part, uint32_t splits,
                                                                uint64_t m, uint64_t n, EpiArgs e) {
    const bool gated = e.act == COEUS_EPI_SILU_GATE;
    const bool vec4 = epi_vec4(e);
    const uint64_t raw_per_thread = gated ? 8 : 4;
    const uint64_t groups = (n + raw_per_thread - 1) / raw_per_thread;  // per row
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= m * groups) return;
    const uint64_t row = gid / groups, raw = (gid - row * groups) * raw_per_thread;
    float v[8];
#pragma unroll
    for (int q = 0; q < 8; q++) v[q] = 0.f;
    const uint64_t plane = m * n;
    if ((n & 3) == 0) {  // (raw + 3 < n: whole groups of 4)
        for (uint32_t s = 0; s < splits; s++) {
            const float *p = part + s * plane + row * n + raw;
            const float4 a = *(const float4 *)p;
            v[0] += a.x; v[1] += a.y; v[2] += a.z; v[3] += a.w;
            if (gated && raw + 7 < n) {
                const float4 c = *(const float4 *)(p + 4);
                v[4] += c.x; v[5] += c.y; v[6] += c.z; v[7] += c.w;
            }
        }
    } else {
        for (uint32_t s = 0; s < splits; s++)
            for (uint64_t q = 0; q < raw_per_thread && raw + q < n; q++) v[q] += part[s * plane + row * n + raw + q];
    }
    if (!gated) {
        float v4[4] = {v[0], v[1], v[2], v[3]};
        epi_row4(e, vec4, epi_kv_cols(e, raw, n), row, raw, n, v4);
    } else {
        const float gv[4] = {v[0], v[2], v[4], v[6]}, uv[4] = {v[1], v[3], v[5], v[7]};
        epi_row4_gated(e, vec4, row, raw >> 1, raw, n, gv, uv);
    }
}

// Which 256x256 output tile the workgroup with number `bid` works on.  Workgroups are numbered so
// that the 32 that run together on one XCD (the hardware deals consecutive workgroups round-robin
// to the 8 XCDs) form a compact block of 4 x 8 output tiles: they walk k in step and share their
// 12 operand tiles through that XCD's L2.
__device__ __forceinline__ void h256_tile_of(uint32_t bid, uint32_t tiles_m, uint32_t tiles_n, uint32_t &tm,
                                             uint32_t &tn) {
    const uint32_t total = tiles_m * tiles_n, per_xcd = total / 8;
    const uint32_t lid = bid < per_xcd * 8 ? (bid % 8) * per_xcd + bid / 8 : bid;
    constexpr uint32_t GM = 4;  // row tiles per group; within a group the order is column-major
    const uint32_t grp = lid / (GM * tiles_n), first_m = grp * GM;
    const uint32_t gsz = min(GM, tiles_m - first_m);
    tm = first_m + (lid % (GM * tiles_n)) % gsz;
    tn = (lid % (GM * tiles_n)) / gsz;
}

// Sums the partial tiles of a launch whose last, incomplete round of tiles was split along k
// ([split][tail tile][256][256] f32) in split order and runs the epilogue.  One thread per 4
// outputs (8 weight rows when gated) of a row; 64 workgroups per tail tile.
__global__ __launch_bounds__(256) void gemm_tail_reduce_kernel(const float *__restrict__ part, uint32_t splits,
                                                               uint32_t full_tiles, uint32_t tiles_m,
                                                               uint32_t tiles_n, uint64_t m, uint64_t n, EpiArgs e) {
    const bool gated = e.act == COEUS_EPI_SILU_GATE;
    const bool vec4 = epi_vec4(e);
    const uint32_t rpt = gated ? 8 : 4, gpr = 256 / rpt;  // raw columns per thread, threads per tile row
    const uint32_t j = blockIdx.x >> 6, within = (blockIdx.x & 63) * 256 + threadIdx.x;
    const uint32_t r = within / gpr, g = within - r * gpr;
    if (r >= 256) return;
    uint32_t tm, tn;
    h256_tile_of(full_tiles + j, tiles_m, tiles_n, tm, tn);
    const uint64_t row = (uint64_t)tm * 256 + r, raw = (uint64_t)tn * 256 + g * rpt;
    if (row >= m || raw >= n) return;
    const uint32_t tail = tiles_m * tiles_n - full_tiles;
    float v[8];
#pragma unroll
    for (int q = 0; q < 8; q++) v[q] = 0.f;
    for (uint32_t s = 0; s < splits; s++) {
        const float *p = part + (((uint64_t)s * tail + j) * 256 + r) * 256 + g * rpt;
        const float4 a = *(const float4 *)p;
        v[0] += a.x; v[1] += a.y; v[2] += a.z; v[3] += a.w;
        if (gated) {
            const float4 c = *(const float4 *)(p + 4);
            v[4] += c.x; v[5] += c.y; v[6] += c.z; v[7] += c.w;
        }
    }
    if (!gated) {
        float v4[4] = {v[0], v[1], v[2], v[3]};
        epi_row4(e, vec4, epi_kv_cols(e, raw, n), row, raw, n, v4);
    } else {
        const float gv[4] = {v[0], v[2], v[4], v[6]}, uv[4] = {v[1], v[3], v[5], v[7]};
        epi_row4_gated(e, vec4, row, raw >> 1, raw, n, gv, uv);
    }
}

// Large-tile variant for k % 32 == 0 (used when k % 64 != 0; gemm_h256k64_kernel below takes the
// others): 256x256 output tile per workgroup, 8 waves of 128x64
// (8 accumulator tiles of 32x32 per wave; two waves per SIMD, so one wave's LDS waits and
// barriers are covered by the other's matrix-core work).  Per 16-wide k step a wave reads 4 + 2
// operand fragments from LDS for 8 matrix-core instructions.
// The 32-wide k slices go from memory straight into LDS (global_load_lds, 16 bytes per lane, no
// register round trip and no LDS store instructions, which were the bottleneck of a
// register-staged version: LDS stores run at a quarter of the read rate).  Four slice buffers:
// a slice is requested three slices before it is used.  Such a load writes the 64 lanes' pieces
// to 1 KiB of consecutive LDS, which fixes the row stride at 64 bytes; the 16-byte pieces of a
// row are therefore stored XOR-swizzled with bits 2-3 of the row index (the loading lane picks
// the global piece that belongs in its slot), which keeps the 32-row fragment reads spread over
// the banks.  One barrier per slice.
// Workgroups are numbered so that the 32 that run together on one XCD (the hardware deals
// consecutive workgroups round-robin to the 8 XCDs) form a compact block of 4 x 8 output tiles:
// they walk k in step and share their 12 operand tiles through that XCD's L2.
constexpr int TM = 256, TN = 256, TK = 32, NSTAGE = 4;

// Requests one slice: 2 + 2 wave instructions of 1 KiB each, straight into LDS.
__device__ __forceinline__ void slice_request(uint16_t *__restrict__ dst, uint32_t wave,
                                              const uint16_t *const (&ag)[2],
                                              const uint16_t *const (&wg)[2], uint64_t k0) {
    typedef const __attribute__((address_space(1))) void *gptr_t;
    typedef __attribute__((address_space(3))) void *lptr_t;
    uint16_t *as_ = dst + (16 * wave) * TK, *ws_ = as_ + TM * TK;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        __builtin_amdgcn_global_load_lds((gptr_t)(ag[i] + k0), (lptr_t)(as_ + 128 * i * TK), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((gptr_t)(wg[i] + k0), (lptr_t)(ws_ + 128 * i * TK), 16, 0, 0);
    }
}

// One slice of matrix-core work on `sb` while a later slice is requested into `dst`.  The two
// buffers are distinct (__restrict__): that is what lets the fragment reads proceed without
// waiting for the loads into `dst` to land.
template <bool BF16>
__device__ __forceinline__ void slice_step(const uint16_t *__restrict__ sb, uint16_t *__restrict__ dst,
                                           uint32_t wave, const uint16_t *const (&ag)[2],
                                           const uint16_t *const (&wg)[2], uint64_t k_next,
                                           const uint32_t (&afo)[4], const uint32_t (&bfo)[2],
                                           uint32_t fhf, uint32_t fsw, float16_t (&acc)[4][2]) {
    typedef const __attribute__((address_space(1))) void *gptr_t;
    typedef __attribute__((address_space(3))) void *lptr_t;
    uint16_t *as_ = dst + (16 * wave) * TK, *ws_ = as_ + TM * TK;
#pragma unroll
    for (int ks = 0; ks < TK; ks += 16) {
        const uint32_t so = 8 * (((ks >> 3) + fhf) ^ fsw);
        uint4 af[4], bf[2];
        // This wave's four requests for the later slice are spread over the slice, one before each
        // half of a k step's products (all four at the top of the slice measured 5 % slower on
        // the FFN-up shape); they have three slices' time to land.
        const int i = ks >> 4;
        __builtin_amdgcn_global_load_lds((gptr_t)(ag[i] + k_next), (lptr_t)(as_ + 128 * i * TK), 16, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int x = 0; x < 4; x++) af[x] = *(const uint4 *)(sb + afo[x] + so);
#pragma unroll
        for (int y = 0; y < 2; y++) bf[y] = *(const uint4 *)(sb + bfo[y] + so);
#pragma unroll
        for (int x = 0; x < 4; x++) {
            if (x == 2) {
                __builtin_amdgcn_sched_barrier(0);
                __builtin_amdgcn_global_load_lds((gptr_t)(wg[i] + k_next), (lptr_t)(ws_ + 128 * i * TK), 16, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
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
}

template <bool BF16>
__global__ __launch_bounds__(512) void gemm_h256_kernel(const uint16_t *a, const uint16_t *w, uint64_t m,
                                                        uint64_t n, uint64_t k, uint64_t lda,
                                                        uint64_t ldw, uint32_t tiles_m,
                                                        uint32_t tiles_n, uint32_t splits, uint32_t full_tiles,
                                                        float *tail_part, EpiArgs e) {
    extern __shared__ __attribute__((aligned(16))) uint16_t sm[];  // [NSTAGE][(TM + TN) * TK]
    constexpr uint32_t BUF = (TM + TN) * TK;
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Three kinds of launch:
    //  * plain (splits == 1): workgroup b computes tile b and runs the epilogue;
    //  * every tile split along k (splits > 1, tail_part == nullptr): workgroup b works on tile
    //    b % total over share b / total of the k slices and stores its bare products into plane
    //    b / total of the buffer that e.out_f32 points to ([split][m][n]);
    //  * only the last, incomplete round of tiles split (tail_part != nullptr): workgroups below
    //    full_tiles are plain; the others take tile full_tiles + j over share s of k and store a
    //    whole 256x256 tile of bare products at tail_part[s][j].
    const uint32_t total = tiles_m * tiles_n;
    uint32_t split = 0, bid = blockIdx.x, shares = 1, tail_idx = 0;
    bool tail_wg = false;
    if (tail_part) {
        if (bid >= full_tiles) {
            const uint32_t tail = total - full_tiles, o = bid - full_tiles;
            split = o / tail;
            tail_idx = o - split * tail;
            bid = full_tiles + tail_idx;
            shares = splits;
            tail_wg = true;
        }
    } else if (splits > 1) {
        split = bid / total;
        bid -= split * total;
        shares = splits;
        e.out_f32 += (uint64_t)split * m * e.n_eff;
    }
    const uint64_t nslices = k / TK;
    const uint64_t kbeg = nslices * split / shares * TK, kend = nslices * (split + 1) / shares * TK;
    uint32_t tm, tn;
    h256_tile_of(bid, tiles_m, tiles_n, tm, tn);
    const uint64_t m0 = (uint64_t)tm * TM, n0 = (uint64_t)tn * TN;
    const uint32_t wm = (wave >> 2) * 128, wn = (wave & 3) * 64;
    float16_t acc[4][2];
#pragma unroll
    for (int x = 0; x < 4; x++)
#pragma unroll
        for (int y = 0; y < 2; y++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[x][y][i] = 0.f;

    // memory -> LDS: a slice is 256 rows x 4 pieces of 16 B per operand.  One wave instruction
    // fills 16 rows (1 KiB); wave v takes rows 16 v + 128 i, lane l row l / 4 of them, slot l % 4,
    // and fetches the piece slot ^ (row / 4 % 4).  Rows past the end are clamped (their results
    // are not stored).
    const uint32_t lr = lane >> 2, lslot = lane & 3;
    const uint16_t *ag[2], *wg[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const uint32_t row = 16 * wave + 128 * i + lr, piece = lslot ^ ((row >> 2) & 3);
        ag[i] = a + (m0 + min((uint64_t)row, m - 1 - m0)) * lda + piece * 8;
        wg[i] = w + (n0 + min((uint64_t)row, n - 1 - n0)) * ldw + piece * 8;
    }
    const uint64_t klast = kend - TK;
    slice_request(sm, wave, ag, wg, kbeg);
    slice_request(sm + BUF, wave, ag, wg, kbeg + TK <= klast ? kbeg + TK : klast);
    slice_request(sm + 2 * BUF, wave, ag, wg, kbeg + 2 * TK <= klast ? kbeg + 2 * TK : klast);
    __builtin_amdgcn_s_waitcnt(0x0078);  // vmcnt(8): slice 0 has landed (this wave's part)
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const uint32_t frow = lane & 31, fhf = lane >> 5;
    // fragment addresses (elements) within a slice buffer: row * 32 + 8 * (piece ^ (row / 4 % 4))
    uint32_t afo[4], bfo[2];
#pragma unroll
    for (int x = 0; x < 4; x++) afo[x] = (wm + x * 32 + frow) * TK;
#pragma unroll
    for (int y = 0; y < 2; y++) bfo[y] = (TM + wn + y * 32 + frow) * TK;
    const uint32_t fsw = (frow >> 2) & 3;  // the same for every fragment row of a lane: tiles start at multiples of 32
    uint32_t st = 0;
    for (uint64_t k0 = kbeg; k0 < kend; k0 += TK) {
        // slice k0 + 3 TK goes into the buffer whose slice (k0 - TK) everybody finished before the
        // last barrier; past the end the last slice is requested again and never used
        slice_step<BF16>(sm + st * BUF, sm + ((st + 3) & (NSTAGE - 1)) * BUF, wave, ag, wg,
                         k0 + 3 * TK <= klast ? k0 + 3 * TK : klast, afo, bfo, fhf, fsw, acc);
        // The next slice has landed (this wave's part: all but the 8 newest loads are done) and
        // this wave's fragment reads are done; then the workgroup barrier.  Not __syncthreads():
        // its fence would wait for every load in flight.
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_s_waitcnt(0x0078);  // vmcnt(8) lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        st = (st + 1) & (NSTAGE - 1);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): nothing may land in LDS once it is reused below

    // Epilogue through LDS (free now): each wave lays one 32-row strip of its 128x64 block at a
    // time out row-major in a private [32][64 + 4] area and walks it with 16-byte accesses: a
    // store instruction covers four 256-byte row segments, and the epilogue is a short loop
    // instead of 128 unrolled scalar copies.
    constexpr uint32_t TS = 68;
    float *strip = (float *)sm + wave * (32 * TS);
    // where the epilogue writes: the output matrix, or (tail workgroups) a private 256x256 tile
    uint64_t em = m, en = n, em0 = m0, en0 = n0;
    if (tail_wg) {
        EpiArgs pe = {};
        pe.out_f32 = tail_part + ((uint64_t)split * (total - full_tiles) + tail_idx) * (TM * TN);
        pe.n = pe.n_eff = TN;
        e = pe;
        em = TM; en = TN; em0 = 0; en0 = 0;
    }
    const bool gated = e.act == COEUS_EPI_SILU_GATE;
    const bool vec4 = epi_vec4(e);
    auto strip_out = [&](const float16_t (&t)[2], uint32_t x) {
#pragma unroll
        for (int y = 0; y < 2; y++)
#pragma unroll
            for (int i = 0; i < 16; i++)
                strip[(8 * (i >> 2) + 4 * (lane >> 5) + (i & 3)) * TS + y * 32 + (lane & 31)] = t[y][i];
        const uint64_t row0 = em0 + wm + x * 32, col0 = en0 + wn;
        if (!gated) {
            const uint32_t c4 = (lane & 15) * 4;
            const KvCols kc = epi_kv_cols(e, col0 + c4, en);
#pragma unroll 2
            for (uint32_t r = lane >> 4; r < 32; r += 4) {
                const uint64_t row = row0 + r, col = col0 + c4;
                const float4 v4 = *(const float4 *)(strip + r * TS + c4);
                float v[4] = {v4.x, v4.y, v4.z, v4.w};
                if (row >= em) continue;
                epi_row4(e, vec4, kc, row, col, en, v);
            }
        } else {
            // weight rows (2c, 2c+1) = (gate_c, up_c): a lane takes 4 outputs = 8 strip columns
            const uint32_t o4 = (lane & 7) * 4;
#pragma unroll 2
            for (uint32_t r = lane >> 3; r < 32; r += 8) {
                const uint64_t row = row0 + r, ocol = (col0 >> 1) + o4;
                const float4 p0 = *(const float4 *)(strip + r * TS + 2 * o4);
                const float4 p1 = *(const float4 *)(strip + r * TS + 2 * o4 + 4);
                const float gv[4] = {p0.x, p0.z, p1.x, p1.z}, uv[4] = {p0.y, p0.w, p1.y, p1.w};
                if (row >= em) continue;
                epi_row4_gated(e, vec4, row, ocol, col0 + 2 * o4, en, gv, uv);
            }
        }
    };
    __syncthreads();  // every wave has finished reading the operand slices, every load has landed
    strip_out(acc[0], 0);
    strip_out(acc[1], 1);
    strip_out(acc[2], 2);
    strip_out(acc[3], 3);
}

// The same 256x256 tile for k % 64 == 0, built around what a CU's shared resources cost per 64 of
// k: 2048 cycles of matrix-core work per SIMD; LDS fragment reads (1024 cycles' worth with eight
// waves of 128x64, 512 with four waves of 128x128); and the path from L2 into LDS, which moves
// whole 128-byte lines whether a request asks for 64 or 128 bytes of them and needs three quarters
// of the matrix-core time for a slice even when nothing else runs.  So: four waves of 128x128
// (16 accumulator tiles each in the accumulation registers, one wave per SIMD), 64-wide k slices,
// loads into LDS that take 8 rows x 128 bytes per wave instruction (full lines), and a schedule
// in which the loads go out one behind every fourth product, all through the slice, each with
// one and a half to two slice times to land.
//
// LDS (160 KiB): three 32-KiB regions for the A rows of a slice, two for the W rows; slice s uses
// A region s % 3 and W region s % 2.  Row stride 128 bytes, the eight 16-byte pieces of a row
// stored at slot = piece ^ (row / 2 % 8) (with row % 8 half of the LDS cycles of the 32-row
// fragment reads are bank conflicts, with row / 2 % 8 none).
//
// A wave keeps the W fragments of the whole slice in registers (4 column blocks x 4 k steps) and
// walks its four 32-row blocks of A one after the other ("step" x: 16 products, 4 k steps x 4
// column blocks, on the A fragments of row block x).  That frees the W region as soon as the
// fragments are read.  One period of the loop runs from the barrier before a slice's last step
// to the next such barrier:
//   step 3 of slice s     reads the A fragments of step 0 and, k step by k step as the old ones
//                         retire, the W fragments of slice s + 1; requests A rows of slice s + 3
//                         into the region that slice s has finished with (barrier 1)
//   step 0 of slice s + 1 reads the A fragments of step 1; the rest of those requests
//   barrier 2             every wave holds the W fragments of slice s + 1: their region is free
//   steps 1 and 2         read the A fragments of steps 2 and 3; request the W rows of slice s + 3
//   barrier 1             behind it the loads of slice s + 2 have landed for every wave (all but
//                         the 16 newest requests of a wave are done)
// Nothing else runs on a wave's SIMD, so every wait is placed where it is already satisfied, and
// the waits are explicit: next to a pending load into LDS the compiler turns a wait for one
// fragment into a wait for all reads.
constexpr int UK = 64;
constexpr uint32_t UREG = 256 * UK;  // elements per region

struct K64Frags {
    uint4 a[2][4];  // [buffer][k step]: the A fragments of one row block
    uint4 b[4][4];  // [column block][k step]: the W fragments of a slice
};

template <bool BF16>
__device__ __forceinline__ void mfma_32x32x16(const uint4 &a, const uint4 &b, float16_t &c) {
    if (BF16) {
        union { uint4 u; bf16x8_t v; } ua, ub;
        ua.u = a; ub.u = b;
        c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ua.v, ub.v, c, 0, 0, 0);
    } else {
        union { uint4 u; half8_t v; } ua, ub;
        ua.u = a; ub.u = b;
        c = __builtin_amdgcn_mfma_f32_32x32x16_f16(ua.v, ub.v, c, 0, 0, 0);
    }
}

// Where the loads of a wave come from: unit 4 q + wave of an operand is 8 rows x 128 bytes; lane
// l takes row l / 8 of them and the piece that belongs in slot l % 8.  Rows past the end are
// clamped (their results are not stored).  The address is a uniform base plus a 32-bit lane
// offset, so a request costs one vector addition between two products.
struct K64Source {
    const char *a, *w;      // tile origins (uniform)
    uint32_t oa[8], ow[8];  // this lane's byte offsets for the wave's eight units of each operand
};

__device__ __forceinline__ void k64_request(const K64Source &src, int q, bool is_w, uint64_t k0, uint16_t *region,
                                            uint32_t wave) {
    typedef const __attribute__((address_space(1))) void *gptr_t;
    typedef __attribute__((address_space(3))) void *lptr_t;
    const char *p = (is_w ? src.w : src.a) + 2 * k0 + (uint64_t)(is_w ? src.ow[q] : src.oa[q]);
    __builtin_amdgcn_global_load_lds((gptr_t)p, (lptr_t)(region + (4 * q + wave) * 512), 16, 0, 0);
}

// Lane constants of the fragment reads (elements): row * 64 + 8 * (piece ^ (row / 2 % 8)) with
// piece = 2 (k step) + lane / 32; a lane's rows are all congruent to lane % 32 modulo 32.
struct K64Lane {
    uint32_t a[4], w[4];  // [k step], row block 0 / column block 0 of the wave
};

__device__ __forceinline__ uint4 k64_read(const uint16_t *region, uint32_t lane_off, int block) {
    return *(const uint4 *)(region + lane_off + block * (32 * UK));
}

// One period (see above).  HEAD: the first slice of a tile: no step 3 in front, the fragments of
// its step 0 and all its W fragments are already in registers.  REQUEST: slice s + 3 exists.
// rd_a / rd_w: regions of slice s + 1; free_a: region of slice s (gets A of s + 3); rd_w is also
// where W of s + 3 goes, after barrier 2: the restrict qualifiers tell the compiler that reads
// never have to wait for loads in flight, which holds because the barriers order them.
template <bool BF16, bool HEAD, bool REQUEST>
__device__ __forceinline__ void k64_period(const uint16_t *__restrict__ rd_a, const uint16_t *__restrict__ rd_w,
                                           uint16_t *__restrict__ free_a, uint16_t *__restrict__ free_w,
                                           const K64Lane &ln, uint32_t wave, const K64Source &src, uint64_t k_req,
                                           K64Frags &f, float16_t (&acc)[4][4]) {
    if (!HEAD) {
        // step 3 of slice s: reads #1-4 A of step 0 (gaps 0-2), #5-17 W of slice s + 1 (gaps 3-15)
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int kk = i >> 2, y = i & 3;
            mfma_32x32x16<BF16>(f.b[y][kk], f.a[1][kk], acc[3][y]);
            if (i == 15) __builtin_amdgcn_s_waitcnt(0xC87F);  // lgkmcnt(8): reads #1-8 (step 0, k step 0) are there
            if (i < 3) f.a[0][i] = k64_read(rd_a, ln.a[i], 0);
            if (i == 2) f.a[0][3] = k64_read(rd_a, ln.a[3], 0);
            if (i >= 3) f.b[(i - 3) & 3][(i - 3) >> 2] = k64_read(rd_w, ln.w[(i - 3) >> 2], (i - 3) & 3);
            if (REQUEST && (i & 3) == 1) k64_request(src, i >> 2, false, k_req, free_a, wave);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // step 0 of slice s + 1: reads #18-20 the last W fragments (gaps 0-2), #21-24 A of step 1 (gaps 3-6)
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const int kk = i >> 2, y = i & 3;
        if (!HEAD && i == 12) {
            __builtin_amdgcn_s_waitcnt(0xC47F);  // lgkmcnt(4): reads #17-20 (k step 3) are there
            __builtin_amdgcn_sched_barrier(0);
            asm volatile("s_nop 0");
        }
        mfma_32x32x16<BF16>(f.b[y][kk], f.a[0][kk], acc[0][y]);
        if (!HEAD && i == 3) __builtin_amdgcn_s_waitcnt(0xC87F);  // lgkmcnt(8): 20 issued, #9-12 (k step 1) are there
        if (!HEAD && i == 6) __builtin_amdgcn_s_waitcnt(0xC77F);  // lgkmcnt(7): 23 issued, #13-16 (k step 2) are there
        if (!HEAD && i < 3) f.b[i + 1][3] = k64_read(rd_w, ln.w[3], i + 1);
        if (i >= 3 && i < 7) f.a[1][i - 3] = k64_read(rd_a, ln.a[i - 3], 1);
        if (REQUEST && !HEAD && (i & 3) == 1) k64_request(src, 4 + (i >> 2), false, k_req, free_a, wave);
        __builtin_amdgcn_sched_barrier(0);
    }
    // barrier 2: every wave has its W fragments of slice s + 1 (it has used them all)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the A fragments of step 1 are there
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const int kk = i >> 2, y = i & 3;
        mfma_32x32x16<BF16>(f.b[y][kk], f.a[1][kk], acc[1][y]);
        if (i < 4) f.a[0][i] = k64_read(rd_a, ln.a[i], 2);
        if (REQUEST && (i & 3) == 1) k64_request(src, i >> 2, true, k_req, free_w, wave);
        __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the A fragments of step 2 are there
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const int kk = i >> 2, y = i & 3;
        mfma_32x32x16<BF16>(f.b[y][kk], f.a[0][kk], acc[2][y]);
        if (i < 4) f.a[1][i] = k64_read(rd_a, ln.a[i], 3);
        if (REQUEST && (i & 3) == 1) k64_request(src, 4 + (i >> 2), true, k_req, free_w, wave);
        __builtin_amdgcn_sched_barrier(0);
    }
    // barrier 1: the A fragments of step 3 are there, so this wave has no read of slice s + 1 in
    // flight; its loads of slice s + 2 have landed (all but this period's 16, or all)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    if (REQUEST) __builtin_amdgcn_s_waitcnt(0x4070);  // vmcnt(16) lgkmcnt(0)
    else __builtin_amdgcn_s_waitcnt(0x0070);          // vmcnt(0) lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    __builtin_amdgcn_sched_barrier(0);
}

// Epilogue: 32 rows x 128 columns of a wave's block at a time go through a private
// [32][128 + 4] LDS area and out in 16-byte accesses (in both directions: the weight fragment is
// the first operand of the products, so a lane holds row lane % 32 of the block and, per register
// group g, the 4 consecutive columns 8 g + 4 (lane / 32) ...).
constexpr uint32_t K64_TS = 132;

__device__ __forceinline__ void k64_strip_write(float *strip, const float16_t (&t)[4], uint32_t lane) {
#pragma unroll
    for (int y = 0; y < 4; y++)
#pragma unroll
        for (int g = 0; g < 4; g++)
            *(float4 *)(strip + (lane & 31) * K64_TS + y * 32 + 8 * g + 4 * (lane >> 5)) =
                make_float4(t[y][4 * g], t[y][4 * g + 1], t[y][4 * g + 2], t[y][4 * g + 3]);
}

// (the 16-bit type is a template parameter: chosen at run time per value, both conversions are
// computed for every value)
template <bool BF16OUT>
__device__ __forceinline__ uint2 k64_pack4(const float (&v)[4]) {
    uint2 p;
    p.x = (uint32_t)f32_to_lp_bits(v[0], BF16OUT) | ((uint32_t)f32_to_lp_bits(v[1], BF16OUT) << 16);
    p.y = (uint32_t)f32_to_lp_bits(v[2], BF16OUT) | ((uint32_t)f32_to_lp_bits(v[3], BF16OUT) << 16);
    return p;
}

// Any epilogue, decided value by value (blocks that end outside the matrix, unusual layouts).
__device__ __forceinline__ void k64_strip_generic(const float *strip, uint32_t lane, const EpiArgs &e, bool gated,
                                                  bool vec4, uint64_t row0, uint64_t col0, uint64_t em, uint64_t en) {
    if (!gated) {
        const uint32_t c4 = (lane & 31) * 4;
        const KvCols kc = epi_kv_cols(e, col0 + c4, en);
#pragma unroll 2
        for (uint32_t r = lane >> 5; r < 32; r += 2) {
            const uint64_t row = row0 + r, col = col0 + c4;
            const float4 v4 = *(const float4 *)(strip + r * K64_TS + c4);
            float v[4] = {v4.x, v4.y, v4.z, v4.w};
            if (row >= em) continue;
            epi_row4(e, vec4, kc, row, col, en, v);
        }
    } else {
        // weight rows (2c, 2c+1) = (gate_c, up_c): a lane takes 4 outputs = 8 strip columns
        const uint32_t o4 = (lane & 15) * 4;
#pragma unroll 2
        for (uint32_t r = lane >> 4; r < 32; r += 4) {
            const uint64_t row = row0 + r, ocol = (col0 >> 1) + o4;
            const float4 p0 = *(const float4 *)(strip + r * K64_TS + 2 * o4);
            const float4 p1 = *(const float4 *)(strip + r * K64_TS + 2 * o4 + 4);
            const float gv[4] = {p0.x, p0.z, p1.x, p1.z}, uv[4] = {p0.y, p0.w, p1.y, p1.w};
            if (row >= em) continue;
            epi_row4_gated(e, vec4, row, ocol, col0 + 2 * o4, en, gv, uv);
        }
    }
}

// The activations of the 16-bit matmuls' fast walks, on the hardware's exp2 and reciprocal (1 ulp
// each; tanhf, expf and the division cost 4-5 times the instructions, and a SiLU-gated block
// evaluates 128 of them per lane): x * sigmoid(x), and 0.5 x (1 + tanh(u)) = x * sigmoid(2 u).
__device__ __forceinline__ float k64_sigmoid(float x) {
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x));
}
__device__ __forceinline__ float k64_silu(float x) { return x * k64_sigmoid(x); }
__device__ __forceinline__ float k64_gelu(float x) {
    const float c0 = 0.7978845608028654f, c1 = 0.044715f;
    return x * k64_sigmoid(2.0f * c0 * x * (1.0f + c1 * x * x));
}

// The common epilogues with every decision made outside the loop over rows (the generic walk
// takes some 400 cycles per 16-byte store, a fifth of a 4096-long tile's time in all).  All 128
// columns of the block lie inside the matrix and 4-column accesses are aligned.  A lane takes
// columns 4 (lane % 32) ... + 3 of rows lane / 32, + 2, ...; the residual values of a strip are
// all requested before its first store goes out (a wait for a load behind a store would wait for
// that store to be acknowledged as well).
template <bool BIAS, bool RES, bool GELU, bool LP, bool BF16OUT = false>
__device__ __forceinline__ void k64_strip_rows(const float *strip, uint32_t lane, const EpiArgs &e, uint64_t row0,
                                               uint64_t col0, uint64_t em) {
    const uint32_t c4 = (lane & 31) * 4, r0 = lane >> 5;
    const uint64_t col = col0 + c4;
    float4 b4 = make_float4(0.f, 0.f, 0.f, 0.f);
    if (BIAS) b4 = *(const float4 *)(e.bias + col);
    const float *sp = strip + r0 * K64_TS + c4;
    const uint64_t ld = LP ? e.lp_ld : e.n_eff;
    uint64_t row = row0 + r0;
    const float *rp = RES ? e.residual + row * e.n_eff + col : nullptr;
    float *of = LP ? nullptr : e.out_f32 + row * ld + col;
    uint16_t *ol = LP ? e.out_lp + row * ld + col : nullptr;
    // groups of 8 rows (the residual values of a group are requested before its stores)
#pragma unroll 1
    for (int jj = 0; jj < 2; jj++) {
        float4 res[8];
        if (RES) {
#pragma unroll
            for (int j = 0; j < 8; j++)
                res[j] = row + 2 * j < em ? *(const float4 *)(rp + (uint64_t)(2 * j) * e.n_eff) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const float4 v4 = *(const float4 *)(sp + 2 * j * K64_TS);
            float v[4] = {v4.x + b4.x, v4.y + b4.y, v4.z + b4.z, v4.w + b4.w};
            if (GELU)
#pragma unroll
                for (int q = 0; q < 4; q++) v[q] = k64_gelu(v[q]);
            if (RES) { v[0] += res[j].x; v[1] += res[j].y; v[2] += res[j].z; v[3] += res[j].w; }
            if (row + 2 * j < em) {
                if (LP) *(uint2 *)(ol + (uint64_t)(2 * j) * ld) = k64_pack4<BF16OUT>(v);
                else *(float4 *)(of + (uint64_t)(2 * j) * ld) = make_float4(v[0], v[1], v[2], v[3]);
            }
        }
        sp += 16 * K64_TS;
        row += 16;
        if (RES) rp += 16 * e.n_eff;
        if (LP) ol += 16 * ld; else of += 16 * ld;
    }
}

// The residual epilogue (h += ...: f32 in, f32 out) of a whole 128x128 block.  Waiting for a
// strip's 16 KiB of residual values strip by strip, each wait behind the previous strip's stores,
// took 60 k cycles per tile, over a third of a 4096-long tile's matmul time.  Here the values of
// strip x + 2 are requested when strip x has been stored, into the registers that strip x's values
// occupied (the fragment registers are free by now), so every request has a strip's time to land
// and no wait for a load is also a wait for younger stores.
template <bool BIAS>
__device__ __forceinline__ void k64_epilogue_residual(float *strip, float16_t (&acc)[4][4], uint32_t lane,
                                                      const EpiArgs &e, uint64_t row0, uint64_t col0, uint64_t em) {
    const uint32_t c4 = (lane & 31) * 4, r0 = lane >> 5;
    const uint64_t col = col0 + c4;
    float4 b4 = make_float4(0.f, 0.f, 0.f, 0.f);
    if (BIAS) b4 = *(const float4 *)(e.bias + col);
    float4 res[2][16];
    auto request = [&](int x, float4 (&r)[16]) {
#pragma unroll
        for (int j = 0; j < 16; j++) {
            const uint64_t row = row0 + 32 * x + r0 + 2 * j;
            r[j] = row < em ? *(const float4 *)(e.residual + row * e.n_eff + col) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    request(0, res[0]);
    request(1, res[1]);
#pragma unroll
    for (int x = 0; x < 4; x++) {
        k64_strip_write(strip, acc[x], lane);
#pragma unroll
        for (int j = 0; j < 16; j++) {
            const uint32_t r = r0 + 2 * j;
            const uint64_t row = row0 + 32 * x + r;
            const float4 v4 = *(const float4 *)(strip + r * K64_TS + c4);
            const float4 q = res[x & 1][j];
            if (row < em)
                *(float4 *)(e.out_f32 + row * e.n_eff + col) =
                    make_float4(v4.x + b4.x + q.x, v4.y + b4.y + q.y, v4.z + b4.z + q.z, v4.w + b4.w + q.w);
        }
        if (x + 2 < 4) request(x + 2, res[x & 1]);
    }
}

// Key / value columns of a prompt pass's q|k|v projection: straight into the cache.
template <bool BIAS, int KVT>  // KVT: COEUS_KV_F32 / F16 / BF16
__device__ __forceinline__ void k64_strip_kv(const float *strip, uint32_t lane, const EpiArgs &e, uint64_t row0,
                                             uint64_t col0, uint64_t em, uint64_t en) {
    const uint32_t c4 = (lane & 31) * 4, r0 = lane >> 5;
    const uint64_t col = col0 + c4;
    const KvCols kc = epi_kv_cols(e, col, en);
    float4 b4 = make_float4(0.f, 0.f, 0.f, 0.f);
    if (BIAS) b4 = *(const float4 *)(e.bias + col);
    // sequence and token of the strip's first row; rows advance by 2 per step
    uint32_t sq = (uint32_t)(row0 + r0) / e.kv_rows_per_seq, tok = (uint32_t)(row0 + r0) - sq * e.kv_rows_per_seq;
#pragma unroll 4
    for (int j = 0; j < 16; j++) {
        const uint32_t r = r0 + 2 * j;
        const float4 v4 = *(const float4 *)(strip + r * K64_TS + c4);
        const float v[4] = {v4.x + b4.x, v4.y + b4.y, v4.z + b4.z, v4.w + b4.w};
        if (row0 + r < em) {
            const uint64_t idx = ((uint64_t)sq * e.kv_heads * e.kv_max_ctx + e.kv_pos0 + tok) * e.kv_hd + kc.off;
            if (KVT == COEUS_KV_F32) *(float4 *)((float *)kc.dst + idx) = make_float4(v[0], v[1], v[2], v[3]);
            else *(uint2 *)((uint16_t *)kc.dst + idx) = k64_pack4<KVT == COEUS_KV_BF16>(v);
        }
        tok += 2;
        while (tok >= e.kv_rows_per_seq) { tok -= e.kv_rows_per_seq; sq++; }
    }
}

// SiLU-gated pairs without bias or residual: weight rows (2c, 2c+1) = (gate_c, up_c); a lane
// takes 4 outputs = 8 strip columns of rows lane / 16, + 4, ...
template <bool LP, bool BF16OUT = false>
__device__ __forceinline__ void k64_strip_gated(const float *strip, uint32_t lane, const EpiArgs &e, uint64_t row0,
                                                uint64_t col0, uint64_t em) {
    const uint32_t o4 = (lane & 15) * 4, r0 = lane >> 4;
    const uint64_t ocol = (col0 >> 1) + o4;
#pragma unroll 4
    for (int j = 0; j < 8; j++) {
        const uint32_t r = r0 + 4 * j;
        const uint64_t row = row0 + r;
        const float4 p0 = *(const float4 *)(strip + r * K64_TS + 2 * o4);
        const float4 p1 = *(const float4 *)(strip + r * K64_TS + 2 * o4 + 4);
        const float v[4] = {k64_silu(p0.x) * p0.y, k64_silu(p0.z) * p0.w, k64_silu(p1.x) * p1.y, k64_silu(p1.z) * p1.w};
        if (row < em) {
            if (LP) *(uint2 *)(e.out_lp + row * e.lp_ld + ocol) = k64_pack4<BF16OUT>(v);
            else *(float4 *)(e.out_f32 + row * e.n_eff + ocol) = make_float4(v[0], v[1], v[2], v[3]);
        }
    }
}

// Which of the walks above serves a wave's block: decided once per block.
enum : uint32_t { K64_GENERIC = 0, K64_ROWS = 1, K64_KV = 2, K64_GATED = 3 };
// for K64_ROWS the low bits of `bits` select bias (1), residual (2), GELU (4), 16-bit output (8)
__device__ __forceinline__ uint32_t k64_epilogue_kind(const EpiArgs &e, bool vec4, uint64_t col0, uint64_t en,
                                                      uint32_t &bits) {
    bits = (e.bias ? 1u : 0u) | (e.residual ? 2u : 0u) | (e.act == COEUS_EPI_GELU ? 4u : 0u) | (e.out_lp ? 8u : 0u);
    const bool one_out = (e.out_f32 != nullptr) != (e.out_lp != nullptr);
    if (!vec4 || col0 + 128 > en || (en & 3)) return K64_GENERIC;
    if (e.act == COEUS_EPI_SILU_GATE) return (!e.bias && !e.residual && one_out) ? K64_GATED : K64_GENERIC;
    if (e.kv_k) {
        if (!e.kv_rows_per_seq || (e.kv_inner & 127)) return K64_GENERIC;
        if (col0 >= e.kv_inner) return K64_KV;
    }
    if (!one_out || (e.residual && e.out_lp) || (bits & 4 && bits & 2)) return K64_GENERIC;
    return K64_ROWS;
}

__device__ __forceinline__ void k64_strip_out(const float *strip, uint32_t lane, const EpiArgs &e, uint32_t kind,
                                              uint32_t bits, bool gated, bool vec4, uint64_t row0, uint64_t col0,
                                              uint64_t em, uint64_t en) {
    if (kind == K64_ROWS) {
        switch (bits) {
        case 0: k64_strip_rows<false, false, false, false>(strip, lane, e, row0, col0, em); break;
        case 1: k64_strip_rows<true, false, false, false>(strip, lane, e, row0, col0, em); break;
        case 2: k64_strip_rows<false, true, false, false>(strip, lane, e, row0, col0, em); break;
        case 3: k64_strip_rows<true, true, false, false>(strip, lane, e, row0, col0, em); break;
        case 4: k64_strip_rows<false, false, true, false>(strip, lane, e, row0, col0, em); break;
        case 5: k64_strip_rows<true, false, true, false>(strip, lane, e, row0, col0, em); break;
        case 8:
            if (e.lp_bf16) k64_strip_rows<false, false, false, true, true>(strip, lane, e, row0, col0, em);
            else k64_strip_rows<false, false, false, true, false>(strip, lane, e, row0, col0, em);
            break;
        case 9:
            if (e.lp_bf16) k64_strip_rows<true, false, false, true, true>(strip, lane, e, row0, col0, em);
            else k64_strip_rows<true, false, false, true, false>(strip, lane, e, row0, col0, em);
            break;
        case 12:
            if (e.lp_bf16) k64_strip_rows<false, false, true, true, true>(strip, lane, e, row0, col0, em);
            else k64_strip_rows<false, false, true, true, false>(strip, lane, e, row0, col0, em);
            break;
        case 13:
            if (e.lp_bf16) k64_strip_rows<true, false, true, true, true>(strip, lane, e, row0, col0, em);
            else k64_strip_rows<true, false, true, true, false>(strip, lane, e, row0, col0, em);
            break;
        default: k64_strip_generic(strip, lane, e, gated, vec4, row0, col0, em, en); break;
        }
    } else if (kind == K64_KV) {
        if (e.kv_dtype == COEUS_KV_F16) {
            if (e.bias) k64_strip_kv<true, COEUS_KV_F16>(strip, lane, e, row0, col0, em, en);
            else k64_strip_kv<false, COEUS_KV_F16>(strip, lane, e, row0, col0, em, en);
        } else if (e.kv_dtype == COEUS_KV_BF16) {
            if (e.bias) k64_strip_kv<true, COEUS_KV_BF16>(strip, lane, e, row0, col0, em, en);
            else k64_strip_kv<false, COEUS_KV_BF16>(strip, lane, e, row0, col0, em, en);
        } else {
            if (e.bias) k64_strip_kv<true, COEUS_KV_F32>(strip, lane, e, row0, col0, em, en);
            else k64_strip_kv<false, COEUS_KV_F32>(strip, lane, e, row0, col0, em, en);
        }
    } else if (kind == K64_GATED) {
        if (!e.out_lp) k64_strip_gated<false>(strip, lane, e, row0, col0, em);
        else if (e.lp_bf16) k64_strip_gated<true, true>(strip, lane, e, row0, col0, em);
        else k64_strip_gated<true, false>(strip, lane, e, row0, col0, em);
    } else {
        k64_strip_generic(strip, lane, e, gated, vec4, row0, col0, em, en);
    }
}

template <bool BF16>
__global__ __launch_bounds__(256) void gemm_h256k64_kernel(const uint16_t *a, const uint16_t *w, uint64_t m,
                                                           uint64_t n, uint64_t k, uint64_t lda,
                                                           uint64_t ldw, uint32_t tiles_m, uint32_t tiles_n,
                                                           uint32_t splits, uint32_t full_tiles,
                                                           float *tail_part, EpiArgs e) {
    extern __shared__ __attribute__((aligned(16))) uint16_t sm[];  // A regions 0-2, W regions 0-1
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // the three kinds of launch of gemm_h256_kernel
    const uint32_t total = tiles_m * tiles_n;
    uint32_t split = 0, bid = blockIdx.x, shares = 1, tail_idx = 0;
    bool tail_wg = false;
    if (tail_part) {
        if (bid >= full_tiles) {
            const uint32_t tail = total - full_tiles, o = bid - full_tiles;
            split = o / tail;
            tail_idx = o - split * tail;
            bid = full_tiles + tail_idx;
            shares = splits;
            tail_wg = true;
        }
    } else if (splits > 1) {
        split = bid / total;
        bid -= split * total;
        shares = splits;
        e.out_f32 += (uint64_t)split * m * e.n_eff;
    }
    const uint64_t nslices = k / UK;
    const uint64_t kbeg = nslices * split / shares * UK, kend = nslices * (split + 1) / shares * UK;
    uint32_t tm, tn;
    h256_tile_of(bid, tiles_m, tiles_n, tm, tn);
    const uint64_t m0 = (uint64_t)tm * TM, n0 = (uint64_t)tn * TN;
    const uint32_t wm = (wave >> 1) * 128, wn = (wave & 1) * 128;
    float16_t acc[4][4];
#pragma unroll
    for (int x = 0; x < 4; x++)
#pragma unroll
        for (int y = 0; y < 4; y++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[x][y][i] = 0.f;

    K64Source src;
    src.a = (const char *)(a + m0 * lda);
    src.w = (const char *)(w + n0 * ldw);
    {
        const uint32_t amax = (uint32_t)min((uint64_t)TM - 1, m - 1 - m0), wmax = (uint32_t)min((uint64_t)TN - 1, n - 1 - n0);
#pragma unroll
        for (int q = 0; q < 8; q++) {
            // row = 8 (4 q + wave) + lane / 8; slot lane % 8 holds piece slot ^ (row / 2 % 8)
            const uint32_t row = 8 * (4 * q + wave) + (lane >> 3), piece = (lane & 7) ^ ((row >> 1) & 7);
            src.oa[q] = min(row, amax) * ((uint32_t)lda * 2) + piece * 16;
            src.ow[q] = min(row, wmax) * ((uint32_t)ldw * 2) + piece * 16;
        }
    }
    K64Lane ln;
    {
        const uint32_t frow = lane & 31, fhf = lane >> 5, fsw = (lane >> 1) & 7;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            ln.a[j] = (wm + frow) * UK + 8 * ((2 * j + fhf) ^ fsw);
            ln.w[j] = (wn + frow) * UK + 8 * ((2 * j + fhf) ^ fsw);
        }
    }
    uint16_t *const rega = sm, *const regw = sm + 3 * UREG;
    auto request_all = [&](uint16_t *region, bool is_w, uint64_t k0) {
#pragma unroll
        for (int q = 0; q < 8; q++) k64_request(src, q, is_w, k0, region, wave);
    };
    // slices past the end are requested as repeats of the last one (and never used), so that the
    // number of loads in flight at each wait does not depend on the number of slices
    const uint64_t klast = kend - UK;
    auto kof = [&](uint64_t j) { return kbeg + j * UK <= klast ? kbeg + j * UK : klast; };
    request_all(rega, false, kbeg);
    request_all(regw, true, kbeg);
    request_all(rega + UREG, false, kof(1));
    request_all(regw + UREG, true, kof(1));
    request_all(rega + 2 * UREG, false, kof(2));
    __builtin_amdgcn_s_waitcnt(0x4F78);  // vmcnt(24): slice 0 has landed (this wave's part)
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    K64Frags f;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        f.a[0][j] = k64_read(rega, ln.a[j], 0);
#pragma unroll
        for (int y = 0; y < 4; y++) f.b[y][j] = k64_read(regw, ln.w[j], y);
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    __builtin_amdgcn_sched_barrier(0);
    // slice 0, steps 0-2; W of slice 2 goes where W of slice 0 was
    const uint64_t nsl = (kend - kbeg) / UK;
    k64_period<BF16, true, true>(rega, regw, nullptr, regw, ln, wave, src, kof(2), f, acc);
    // periods s = 0 .. nsl - 2: the last step of slice s and steps 0-2 of slice s + 1
    uint32_t ra = 0, rw = 0;  // regions of slice s
    uint64_t s = 0;
    for (; s + 3 < nsl; s++) {
        const uint32_t ra1 = ra == 2 ? 0 : ra + 1;
        k64_period<BF16, false, true>(rega + ra1 * UREG, regw + (rw ^ 1) * UREG, rega + ra * UREG,
                                      regw + (rw ^ 1) * UREG, ln, wave, src, kbeg + (s + 3) * UK, f, acc);
        ra = ra1;
        rw ^= 1;
    }
    for (; s + 1 < nsl; s++) {
        const uint32_t ra1 = ra == 2 ? 0 : ra + 1;
        k64_period<BF16, false, false>(rega + ra1 * UREG, regw + (rw ^ 1) * UREG, nullptr, nullptr, ln, wave, src, 0,
                                       f, acc);
        ra = ra1;
        rw ^= 1;
    }
    // the last step of the last slice
#pragma unroll
    for (int i = 0; i < 16; i++) mfma_32x32x16<BF16>(f.b[i & 3][i >> 2], f.a[1][i >> 2], acc[3][i & 3]);
    __builtin_amdgcn_s_waitcnt(0x0070);

    // Epilogue through LDS (free now), one 32-row strip of the wave's 128x128 block at a time.
    float *strip = (float *)sm + wave * (32 * 132);
    uint64_t em = m, en = n, em0 = m0, en0 = n0;
    if (tail_wg) {
        EpiArgs pe = {};
        pe.out_f32 = tail_part + ((uint64_t)split * (total - full_tiles) + tail_idx) * (TM * TN);
        pe.n = pe.n_eff = TN;
        e = pe;
        em = TM; en = TN; em0 = 0; en0 = 0;
    }
    const bool gated = e.act == COEUS_EPI_SILU_GATE;
    const bool vec4 = epi_vec4(e);
    uint32_t bits;
    const uint32_t kind = k64_epilogue_kind(e, vec4, en0 + wn, en, bits);
    __syncthreads();  // every wave has finished reading the operand slices
    if (kind == K64_ROWS && (bits & ~1u) == 2) {
        if (bits & 1) k64_epilogue_residual<true>(strip, acc, lane, e, em0 + wm, en0 + wn, em);
        else k64_epilogue_residual<false>(strip, acc, lane, e, em0 + wm, en0 + wn, em);
        return;
    }
    // one copy of the walks for the four row blocks; the accumulators are named with constant
    // indices (indexed dynamically they would live in scratch memory)
#pragma unroll 1
    for (uint32_t x = 0; x < 4; x++) {
        if (x == 0) k64_strip_write(strip, acc[0], lane);
        else if (x == 1) k64_strip_write(strip, acc[1], lane);
        else if (x == 2) k64_strip_write(strip, acc[2], lane);
        else k64_strip_write(strip, acc[3], lane);
        k64_strip_out(strip, lane, e, kind, bits, gated, vec4, em0 + wm + x * 32, en0 + wn, em, en);
    }
}

// Any number of rows: a short prompt leaves most of a 256-row tile empty (rows past the end are
// clamped on the way in and not stored), and is still several times faster here than in the
// 128x128 register-staged kernel (1B shape, 16 rows: 24.5 ms per prompt pass there).
static bool gemm_uses_h256(const Weight &w, uint64_t m) {
    return w.dtype != COEUS_W_F32 && (w.k % TK) == 0 && m >= 1 && w.n >= 128 &&
           (uint64_t)TM * gemm_ld(w.k) < (1ull << 31);  // the byte offsets within a tile fit 32 bits
}

// A launch of few tiles (short prompts, narrow matrices) leaves most CUs without a workgroup while
// each tile walks all of k at about a microsecond per 32-wide slice.  Such launches are split along
// k: `splits` workgroups per tile each take a share of the slices and store plain partial products,
// and a second kernel sums them in split order (deterministic) and runs the epilogue.  At least 8
// slices per split (the request pipeline is 3 deep), at most 16 splits (each adds a plane of
// m x n floats to write and read back), no more workgroups than CUs (one workgroup fills a CU's LDS).
static uint32_t gemm_splits_wanted(const Weight &w, uint64_t m) {
    if (!gemm_uses_h256(w, m)) return 1;
    const uint64_t tiles = ceil_div(m, TM) * ceil_div(w.n, TN), slices = w.k / TK;
    if (tiles > 128) return 1;
    uint64_t s = 256 / tiles;
    if (s > slices / 8) s = slices / 8;
    if (s > 16) s = 16;
    return s < 2 ? 1 : (uint32_t)s;
}

// A larger launch runs its tiles in rounds of 256 (one workgroup fills a CU), and the last round
// is rarely full: 1376 tiles are five rounds and 96 tiles, which take as long as a sixth round.
// When that remainder is at most half a round its tiles alone are split along k (as many shares
// as fit in one round), through private 256x256 partial tiles and gemm_tail_reduce_kernel.
// Returns the number of shares (1: no split) and the number of tiles of the complete rounds.
static uint32_t gemm_tail_splits_wanted(const Weight &w, uint64_t m, uint32_t *full_tiles) {
    *full_tiles = 0;
    if (!gemm_uses_h256(w, m)) return 1;
    const uint64_t tiles = ceil_div(m, TM) * ceil_div(w.n, TN), slices = w.k / TK;
    const uint64_t full = tiles / 256 * 256, tail = tiles - full;
    if (full == 0 || tail == 0 || tail > 128 || tiles > 0xffffffffull / 16) return 1;
    uint64_t s = 256 / tail;
    if (s > slices / 8) s = slices / 8;
    if (s > 16) s = 16;
    if (s < 2) return 1;
    *full_tiles = (uint32_t)full;
    return (uint32_t)s;
}

uint64_t gemm_split_scratch_bytes(const Weight &w, uint64_t m) {
    if (w.dtype == COEUS_W_F32) {
        const uint32_t sf = gemm_f32_splits_wanted(w, m);
        return sf > 1 ? (uint64_t)sf * m * w.n * 4 : 0;
    }
    if (gemm_uses_qskinny(w, m)) return gemm_qskinny_scratch_bytes(w, m);
    const uint32_t s = gemm_splits_wanted(w, m);
    if (s > 1) return (uint64_t)s * m * w.n * 4;
    uint32_t full = 0;
    const uint32_t st = gemm_tail_splits_wanted(w, m, &full);
    if (st > 1) return (uint64_t)st * (ceil_div(m, TM) * ceil_div(w.n, TN) - full) * TM * TN * 4;
    return 0;
}

bool gemm_appends_kv(const Weight &w, uint64_t m, uint64_t inner, uint64_t hd) {
    // rows fit 32 bits; a lane's 4 columns stay inside one head.  (The short-prompt kernel for
    // quantised weights qualifies when it is split along k: the kernel that sums its partial
    // planes runs this same epilogue.)
    return gemm_uses_h256(w, m) && (!gemm_uses_qskinny(w, m) || gemm_qskinny_scratch_bytes(w, m) > 0) && m < (1ull << 32) && w.n == 3 * inner && (inner & 3) == 0 && (hd & 3) == 0;
}

int launch_gemm(const Weight &w, const void *a_in, uint64_t m, const Epilogue &ep, GemmScratch &scr,
                hipStream_t st, bool a_staged) {
    const float *a = (const float *)a_in;
    if (m == 0) return fail(COEUS_INVALID_INPUT, "matmul with zero rows");
    if (ep.act == COEUS_EPI_SILU_GATE && (w.n & 1))
        return fail(COEUS_INVALID_INPUT, "gated epilogue needs an even number of weight rows");
    if (ep.out_xq) return fail(COEUS_INVALID_INPUT, "prefill matmul has no xq output");
    if (w.dtype == COEUS_W_F32) {
        if (a_staged) return fail(COEUS_INVALID_INPUT, "f32 weights take f32 activations");
        return launch_gemm_f32(w, a, m, ep, scr, st);
    }
    const uint64_t lda = gemm_ld(w.k), a_bytes = m * lda * 2;
    const uint16_t *wp = (const uint16_t *)w.data;
    const bool bf = w.dtype == COEUS_W_BF16;
    uint64_t ldw = w.k;
    const uint16_t *ap = (const uint16_t *)a_in;
    if (!a_staged) {
        if (!scr.a_lp || scr.a_lp_bytes < a_bytes)
            return fail(COEUS_INVALID_INPUT, "matmul staging buffer too small (%llu < %llu bytes)",
                        (unsigned long long)scr.a_lp_bytes, (unsigned long long)a_bytes);
        COEUS_TRY(launch_f32_to_16(a, scr.a_lp, m, w.k, lda, bf, st));
        ap = (const uint16_t *)scr.a_lp;
    }
    const uint64_t qs_bytes = gemm_uses_qskinny(w, m) ? gemm_qskinny_scratch_bytes(w, m) : 0;
    if (gemm_uses_qskinny(w, m) && (qs_bytes ? scr.partials && scr.partials_bytes >= qs_bytes : !ep.kv_rows_per_seq)) {
        // up to 64 rows on quantised weights: the kernel that streams the quantised blocks
        const EpiArgs e = make_epi(ep, w.n);
        if (scr.ev_begin) COEUS_HIP(hipEventRecord(scr.ev_begin, st));
        for (uint32_t rep = 0; rep < (scr.repeat ? scr.repeat : 1); rep++) {
            uint32_t splits = 1;
            COEUS_TRY(launch_gemm_qskinny(w, ap, lda, m, e, scr.partials, scr.partials_bytes, &splits, st));
            if (splits > 1) {
                const uint64_t groups = ceil_div(w.n, e.act == COEUS_EPI_SILU_GATE ? 8 : 4);
                hipLaunchKernelGGL(gemm_split_reduce_kernel, dim3((unsigned)ceil_div(m * groups, 256)), dim3(256), 0, st,
                                   (const float *)scr.partials, splits, m, w.n, e);
            }
        }
        if (scr.ev_end) COEUS_HIP(hipEventRecord(scr.ev_end, st));
        COEUS_HIP(hipGetLastError());
        return COEUS_OK;
    }
    if (!bf) {
        ldw = gemm_ld(w.k);
        const uint64_t w_bytes = w.n * ldw * 2;
        if (!w.expanded) COEUS_TRY(weight_expand(w, scr.expand_budget, st));
        if (w.expanded) {
            wp = (const uint16_t *)w.expanded;
        } else {
            if (!scr.w_lp || scr.w_lp_bytes < w_bytes)
                return fail(COEUS_INVALID_INPUT, "weight staging buffer too small (%llu < %llu bytes)",
                            (unsigned long long)scr.w_lp_bytes, (unsigned long long)w_bytes);
            COEUS_TRY(launch_dequant_to_f16(w, (__half *)scr.w_lp, ldw, st));
            wp = (const uint16_t *)scr.w_lp;
        }
    }
    const EpiArgs e = make_epi(ep, w.n);
    if (ep.kv_rows_per_seq && !gemm_appends_kv(w, m, ep.kv_inner, ep.kv_hd))
        return fail(COEUS_INVALID_INPUT, "this matmul cannot append to the cache (see gemm_appends_kv)");
    if (gemm_uses_h256(w, m)) {
        const size_t lds = (size_t)NSTAGE * (TM + TN) * TK * 2, lds64 = (size_t)5 * UREG * 2;
        static const bool once = [] {
            (void)hipFuncSetAttribute((const void *)gemm_h256_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void *)gemm_h256_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void *)gemm_h256k64_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void *)gemm_h256k64_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            return true;
        }();
        (void)once;
        const uint32_t tiles_m = (uint32_t)ceil_div(m, TM), tiles_n = (uint32_t)ceil_div(w.n, TN);
        // split along k (every tile, or the tiles of the last round) when the caller's scratch has
        // room for the partial products
        uint32_t splits = gemm_splits_wanted(w, m), full_tiles = 0, tail_splits = 1;
        if (splits > 1 && (!scr.partials || scr.partials_bytes < (uint64_t)splits * m * w.n * 4)) splits = 1;
        if (splits == 1) {
            tail_splits = gemm_tail_splits_wanted(w, m, &full_tiles);
            if (tail_splits > 1 && (!scr.partials || scr.partials_bytes < gemm_split_scratch_bytes(w, m)))
                tail_splits = 1;
        }
        const uint32_t tail_tiles = tail_splits > 1 ? tiles_m * tiles_n - full_tiles : 0;
        float *tail_part = tail_splits > 1 ? scr.partials : nullptr;
        const dim3 grid(tail_splits > 1 ? full_tiles + tail_tiles * tail_splits : tiles_m * tiles_n * splits);
        const uint32_t ksplits = tail_splits > 1 ? tail_splits : splits;
        EpiArgs plain;  // the split kernels store bare products: [split][m][n] f32
        if (splits > 1) {
            Epilogue pe;
            pe.out_f32 = scr.partials;
            plain = make_epi(pe, w.n);
        }
        const EpiArgs &ke = splits > 1 ? plain : e;
        const uint64_t groups = ceil_div(w.n, e.act == COEUS_EPI_SILU_GATE ? 8 : 4);
        if (scr.ev_begin) COEUS_HIP(hipEventRecord(scr.ev_begin, st));
        for (uint32_t rep = 0; rep < (scr.repeat ? scr.repeat : 1); rep++) {
            if (w.k % UK == 0 && bf)
                hipLaunchKernelGGL(gemm_h256k64_kernel<true>, grid, dim3(256), lds64, st, ap, wp, m, w.n, w.k, lda, ldw, tiles_m, tiles_n, ksplits, full_tiles, tail_part, ke);
            else if (w.k % UK == 0)
                hipLaunchKernelGGL(gemm_h256k64_kernel<false>, grid, dim3(256), lds64, st, ap, wp, m, w.n, w.k, lda, ldw, tiles_m, tiles_n, ksplits, full_tiles, tail_part, ke);
            else if (bf)
                hipLaunchKernelGGL(gemm_h256_kernel<true>, grid, dim3(512), lds, st, ap, wp, m, w.n, w.k, lda, ldw, tiles_m, tiles_n, ksplits, full_tiles, tail_part, ke);
            else
                hipLaunchKernelGGL(gemm_h256_kernel<false>, grid, dim3(512), lds, st, ap, wp, m, w.n, w.k, lda, ldw, tiles_m, tiles_n, ksplits, full_tiles, tail_part, ke);
            if (splits > 1)
                hipLaunchKernelGGL(gemm_split_reduce_kernel, dim3((unsigned)ceil_div(m * groups, 256)), dim3(256), 0, st,
                                   (const float *)scr.partials, splits, m, w.n, e);
            if (tail_splits > 1)
                hipLaunchKernelGGL(gemm_tail_reduce_kernel, dim3(tail_tiles * 64), dim3(256), 0, st,
                                   (const float *)scr.partials, tail_splits, full_tiles, tiles_m, tiles_n, m, w.n, e);
        }
        if (scr.ev_end) COEUS_HIP(hipEventRecord(scr.ev_end, st));
        COEUS_HIP(hipGetLastError());
        return COEUS_OK;
    }
    const dim3 grid((unsigned)ceil_div(w.n, HN), (unsigned)ceil_div(m, HM));
    if (scr.ev_begin) COEUS_HIP(hipEventRecord(scr.ev_begin, st));
    for (uint32_t rep = 0; rep < (scr.repeat ? scr.repeat : 1); rep++) {
        if (bf)
            hipLaunchKernelGGL(gemm_h_kernel<true>, grid, dim3(256), 0, st, ap, wp, m, w.n, w.k, lda, ldw, e);
        else
            hipLaunchKernelGGL(gemm_h_kernel<false>, grid, dim3(256), 0, st, ap, wp, m, w.n, w.k, lda, ldw, e);
    }
    if (scr.ev_end) COEUS_HIP(hipEventRecord(scr.ev_end, st));
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

}  // namespace coeus
