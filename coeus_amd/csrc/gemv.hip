// Decode matmul: y[b, :] = x[b, :] . W for b < batch <= 16 (math::matmul, MT:50-74, with
// m = batch), the HBM-bound kernel of token generation.
//
//   gemv_quant_kernel  Q8_0 / Q4_0 weights in MFMA-native tiles.  One workgroup owns a tile of
//                      16 output rows; its waves take interleaved 128-k chunks (1 KiB of Q4_0
//                      quants = one fully coalesced 16 B/lane load per wave).  Each 32-k block
//                      is one v_mfma_f32_16x16x32_f16 between up to 16 activation rows (f16) and
//                      the block's integers (q-8 resp. q, exact in f16); the f32 block result is
//                      scaled by the block's f16 scale on the VALU, so the value used for every
//                      weight is exactly its dequantised value q*d.
//   gemv_dense_kernel  f32 / bf16 weights, one wave per output row, f32 FMA on the VALU.
#include "device_utils.hpp"

namespace coeus {

// ---------------------------------------------------------------- xq packing
__global__ void pack_xq_kernel(const float *x, uint32_t batch, uint32_t bp, uint64_t k,
                               uint64_t k_pad, __half *xq) {
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= k_pad * bp) return;
    const uint32_t e = idx & 7, b = (idx >> 3) % bp;
    const uint64_t kk = (idx >> 3) / bp * 8 + e;
    const float v = (b < batch && kk < k) ? x[(uint64_t)b * k + kk] : 0.0f;
    xq[idx] = __float2half_rn(v);
}

int launch_pack_xq(const float *x, uint64_t batch, uint64_t k, uint64_t k_pad, __half *xq,
                   hipStream_t st) {
    const uint32_t bp = pad_batch(batch);
    hipLaunchKernelGGL(pack_xq_kernel, dim3((unsigned)ceil_div(k_pad * bp, 256)), dim3(256), 0, st,
                       x, (uint32_t)batch, bp, k, k_pad, xq);
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

// ---------------------------------------------------------------- quantised kernel
// Q4_0 dword (nibble positions [k0,k2,k4,k6,k1,k3,k5,k7]) -> 8 f16 values q-8, exact:
// 0x6400|n is the f16 1024+n; 0x6400|(n<<4) is 1024+16n, and (1024+16n)/16 - 72 = n - 8.
__device__ __forceinline__ half8_t unpack_q4(uint32_t q) {
    const uint32_t q8 = q >> 8;
    union { uint32_t u; half2_t h; } a, b, c, d;
    a.u = (q & 0x000F000Fu) | 0x64006400u;
    b.u = (q & 0x00F000F0u) | 0x64006400u;
    c.u = (q8 & 0x000F000Fu) | 0x64006400u;
    d.u = (q8 & 0x00F000F0u) | 0x64006400u;
    const half2_t off_lo = {(_Float16)1032.0f, (_Float16)1032.0f};
    const half2_t sc_hi = {(_Float16)0.0625f, (_Float16)0.0625f};
    const half2_t off_hi = {(_Float16)72.0f, (_Float16)72.0f};
    const half2_t r0 = a.h - off_lo, r1 = b.h * sc_hi - off_hi;
    const half2_t r2 = c.h - off_lo, r3 = d.h * sc_hi - off_hi;
    half8_t out = {r0.x, r0.y, r1.x, r1.y, r2.x, r2.y, r3.x, r3.y};
    return out;
}

// Two dwords of int8 -> 8 f16, exact: byte^0x80 = q+128; 0x6400|(q+128) = 1152+q.
__device__ __forceinline__ half8_t unpack_q8(uint32_t lo, uint32_t hi) {
    const uint32_t l = lo ^ 0x80808080u, h = hi ^ 0x80808080u;
    union { uint32_t u; half2_t h2; } a, b, c, d;
    a.u = __builtin_amdgcn_perm(0x64646464u, l, 0x04010400u);
    b.u = __builtin_amdgcn_perm(0x64646464u, l, 0x04030402u);
    c.u = __builtin_amdgcn_perm(0x64646464u, h, 0x04010400u);
    d.u = __builtin_amdgcn_perm(0x64646464u, h, 0x04030402u);
    const half2_t off = {(_Float16)1152.0f, (_Float16)1152.0f};
    const half2_t r0 = a.h2 - off, r1 = b.h2 - off, r2 = c.h2 - off, r3 = d.h2 - off;
    half8_t out = {r0.x, r0.y, r1.x, r1.y, r2.x, r2.y, r3.x, r3.y};
    return out;
}

// One chunk = 16 rows x 128 k.  Matrix-core roles: A = activations (row = batch entry),
// B = weights (column = weight row), so lane (j = lane%16, ig = lane/16) ends up holding the
// results of weight row j for batch entries 4*ig..4*ig+3, and a block's scale is ONE value per
// lane.  Activations come from LDS when the whole reduction run fits (staged once per
// workgroup, overlapped with the first weight loads), from global memory (L2) otherwise.
template <bool Q4>
struct ChunkRegs {
    uint4 q0, q1;  // q1 only for Q8_0
    uint2 s;       // the lane's row: 4 block scales (f16)
};

template <bool Q4>
__device__ __forceinline__ void load_chunk(ChunkRegs<Q4> &r, const uint4 *__restrict__ qs,
                                           const uint2 *__restrict__ ds, uint64_t chunk,
                                           uint32_t lane) {
    if (Q4) {
        r.q0 = load_stream(qs + chunk * 64 + lane);
    } else {
        r.q0 = load_stream(qs + (chunk * 2) * 64 + lane);
        r.q1 = load_stream(qs + (chunk * 2 + 1) * 64 + lane);
    }
    r.s = ds[chunk * 16 + (lane & 15)];
}

// How the activation block reaches the matrix cores.
enum { X_GLOBAL = 0,  // xq read from global memory (L2) per block: no LDS needed, any size
       X_LDS = 1,     // xq copied into LDS once per workgroup
       X_LAYERNORM = 2, X_RMSNORM = 3 };  // f32 residual rows normalised while staged into LDS

struct XArgs {
    const uint4 *xq;     // X_GLOBAL / X_LDS
    const float *h;      // X_*NORM: [batch, k]
    const float *nscale, *nbias;
    float eps;
    uint32_t k;          // logical reduction length
};

// Fills smem (xq order, [k_pad/8][BP] pieces of 8 f16) with norm(h).  Every thread keeps its
// pieces (8 consecutive k of one row) in registers: h is read from memory once, the per-row
// statistics come from block reductions, and y = scale * (x - mean) / sd + bias is evaluated
// exactly as norm_token_kernel does.  At most NORM_PPT pieces per thread.
constexpr int NORM_PPT = 4;

template <int BP>
__device__ __forceinline__ void block_sums(float (&s)[BP], float *red) {
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
#pragma unroll
    for (int b = 0; b < BP; b++) s[b] = wave_sum(s[b]);
    __syncthreads();  // red may still be read from the previous reduction
    if (lane == 0)
#pragma unroll
        for (int b = 0; b < BP; b++) red[wave * BP + b] = s[b];
    __syncthreads();
#pragma unroll
    for (int b = 0; b < BP; b++) {
        float t = 0.f;
        for (uint32_t w = 0; w < nw; w++) t += red[w * BP + b];
        s[b] = t;
    }
}

template <int BP, bool RMS>
__device__ __forceinline__ void stage_normed(uint4 *smem, float *red, const XArgs &xa,
                                             uint32_t batch, uint32_t ngroups) {
    const uint32_t tid = threadIdx.x, nth = blockDim.x, k = xa.k;
    const uint32_t total = ngroups * 16 * BP;  // pieces, index p = (k/8)*BP + b
    float v[NORM_PPT][8];
    float sum[BP];
#pragma unroll
    for (int b = 0; b < BP; b++) sum[b] = 0.f;
#pragma unroll
    for (int t = 0; t < NORM_PPT; t++) {
        const uint32_t p = tid + t * nth, b = p % BP, kk = (p / BP) * 8;
        const bool live = p < total && b < batch && kk < k;  // k % 32 == 0: all in or all out
        if (live) {
            const float4 a0 = *(const float4 *)(xa.h + (uint64_t)b * k + kk);
            const float4 a1 = *(const float4 *)(xa.h + (uint64_t)b * k + kk + 4);
            v[t][0] = a0.x; v[t][1] = a0.y; v[t][2] = a0.z; v[t][3] = a0.w;
            v[t][4] = a1.x; v[t][5] = a1.y; v[t][6] = a1.z; v[t][7] = a1.w;
        } else {
#pragma unroll
            for (int u = 0; u < 8; u++) v[t][u] = 0.f;
        }
        if (!RMS) {
            float ps = 0.f;
#pragma unroll
            for (int u = 0; u < 8; u++) ps += v[t][u];
#pragma unroll
            for (int bb = 0; bb < BP; bb++) sum[bb] += (live && b == (uint32_t)bb) ? ps : 0.f;
        }
    }
    float mean[BP];
    if (!RMS) {
        block_sums<BP>(sum, red);
#pragma unroll
        for (int b = 0; b < BP; b++) mean[b] = sum[b] / (float)k;
    } else {
#pragma unroll
        for (int b = 0; b < BP; b++) mean[b] = 0.f;
    }
#pragma unroll
    for (int b = 0; b < BP; b++) sum[b] = 0.f;
#pragma unroll
    for (int t = 0; t < NORM_PPT; t++) {
        const uint32_t p = tid + t * nth, b = p % BP, kk = (p / BP) * 8;
        const bool live = p < total && b < batch && kk < k;
        float mb = 0.f;
#pragma unroll
        for (int bb = 0; bb < BP; bb++) mb = b == (uint32_t)bb ? mean[bb] : mb;
        float ps = 0.f;
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const float d = v[t][u] - mb;
            ps = fmaf(d, d, ps);
        }
#pragma unroll
        for (int bb = 0; bb < BP; bb++) sum[bb] += (live && b == (uint32_t)bb) ? ps : 0.f;
    }
    block_sums<BP>(sum, red);
    float sd[BP];
#pragma unroll
    for (int b = 0; b < BP; b++) sd[b] = sqrtf(sum[b] / (float)k + xa.eps);
#pragma unroll
    for (int t = 0; t < NORM_PPT; t++) {
        const uint32_t p = tid + t * nth, b = p % BP, kk = (p / BP) * 8;
        if (p >= total) continue;
        union { uint4 u; half2_t h2[4]; } o;
        o.u = make_uint4(0, 0, 0, 0);
        if (b < batch && kk < k) {
            float mb = 0.f, sb = 1.f;
#pragma unroll
            for (int bb = 0; bb < BP; bb++) { mb = b == (uint32_t)bb ? mean[bb] : mb; sb = b == (uint32_t)bb ? sd[bb] : sb; }
            const float4 s0 = *(const float4 *)(xa.nscale + kk), s1 = *(const float4 *)(xa.nscale + kk + 4);
            const float sc[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
            float y[8];
#pragma unroll
            for (int u = 0; u < 8; u++) y[u] = sc[u] * (v[t][u] - mb) / sb;
            if (!RMS) {
                const float4 b0 = *(const float4 *)(xa.nbias + kk), b1 = *(const float4 *)(xa.nbias + kk + 4);
                const float bi[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
#pragma unroll
                for (int u = 0; u < 8; u++) y[u] += bi[u];
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                o.h2[u].x = (_Float16)y[2 * u];
                o.h2[u].y = (_Float16)y[2 * u + 1];
            }
        }
        smem[p] = o.u;
    }
    __syncthreads();
}

template <bool Q4, int BP, int XMODE>
__global__ __launch_bounds__(1024) void gemv_quant_kernel(const uint4 *__restrict__ qs,
                                                          const uint2 *__restrict__ ds, XArgs xa,
                                                          uint32_t ngroups, uint32_t batch,
                                                          EpiArgs e) {
    constexpr int NI = BP < 4 ? BP : 4;  // accumulator rows that can hold a real batch entry
    constexpr bool XLDS = XMODE != X_GLOBAL;
    extern __shared__ uint4 smem[];      // [x: ngroups*16*BP uint4 if XLDS][reduction]
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    const uint32_t T = blockIdx.x;
    const uint32_t g = lane >> 4, xb = (lane & 15) & (BP - 1);
    float acc[NI];
#pragma unroll
    for (int i = 0; i < NI; i++) acc[i] = 0.f;
    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
    const uint4 *__restrict__ xq = xa.xq;

    // PF chunks (PF KiB of Q4_0 quants per wave) are requested before any of them is used:
    // with ~24 waves per CU that keeps enough bytes in flight to cover HBM latency.
    constexpr int PF = Q4 ? 4 : 2;  // the same bytes in flight for both formats
    const uint32_t nx = ngroups * 16 * BP;  // uint4 pieces of the activation block
    float *red = (float *)(smem + (XLDS ? nx : 0));
    bool staged = !XLDS;
    auto stage = [&]() {
        if (XMODE == X_LDS) {
            for (uint32_t i = threadIdx.x; i < nx; i += blockDim.x) smem[i] = xq[i];
            __syncthreads();
        } else if (XMODE == X_LAYERNORM) {
            stage_normed<BP, false>(smem, red, xa, batch, ngroups);
        } else if (XMODE == X_RMSNORM) {
            stage_normed<BP, true>(smem, red, xa, batch, ngroups);
        }
    };
    for (uint32_t G0 = wave; G0 < ngroups; G0 += nwaves * PF) {
        ChunkRegs<Q4> r[PF];
#pragma unroll
        for (int u = 0; u < PF; u++) {
            const uint32_t G = G0 + u * nwaves;
            if (G < ngroups) load_chunk<Q4>(r[u], qs, ds, (uint64_t)T * ngroups + G, lane);
        }
        if (!staged) {  // first pass only; uniform across the workgroup
            stage();
            staged = true;
        }
#pragma unroll
        for (int u = 0; u < PF; u++) {
            const uint32_t G = G0 + u * nwaves;
            if (G >= ngroups) break;
            const uint32_t qw[8] = {r[u].q0.x, r[u].q0.y, r[u].q0.z, r[u].q0.w,
                                    Q4 ? 0u : r[u].q1.x, Q4 ? 0u : r[u].q1.y, Q4 ? 0u : r[u].q1.z,
                                    Q4 ? 0u : r[u].q1.w};
            union { uint2 u2; half2_t h[2]; } sc;
            sc.u2 = r[u].s;
            const float d[4] = {(float)sc.h[0].x, (float)sc.h[0].y, (float)sc.h[1].x, (float)sc.h[1].y};
#pragma unroll
            for (int jj = 0; jj < 4; jj++) {
                const uint32_t xi = ((G * 4 + jj) * 4 + g) * BP + xb;
                union { uint4 u4; half8_t h; } xv;
                xv.u4 = XLDS ? smem[xi] : xq[xi];
                const half8_t wv = Q4 ? unpack_q4(qw[jj]) : unpack_q8(qw[2 * jj], qw[2 * jj + 1]);
                const float4_t part = __builtin_amdgcn_mfma_f32_16x16x32_f16(xv.h, wv, zero, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < NI; i++) acc[i] = fmaf(d[jj], part[i], acc[i]);
            }
        }
    }
    if (!staged) stage();  // a wave without chunks still takes part in the staging

    // deterministic cross-wave reduction (fixed order), then the epilogue on wave 0
    if (nwaves > 1) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < NI; i++) red[(wave * NI + i) * 64 + lane] = acc[i];
        __syncthreads();
        if (wave != 0) return;
        for (uint32_t w = 1; w < nwaves; w++)
#pragma unroll
            for (int i = 0; i < NI; i++) acc[i] += red[(w * NI + i) * 64 + lane];
    }
    const uint64_t j = (uint64_t)T * 16 + (lane & 15);
    const bool gated = e.act == COEUS_EPI_SILU_GATE;
#pragma unroll
    for (int i = 0; i < NI; i++) {
        const uint32_t b = 4 * g + i;
        // gated: weight rows (2m, 2m+1) = (gate_m, up_m) sit in neighbouring lanes
        const float other = __shfl_xor(acc[i], 1, 64);
        if (b >= batch || j >= e.n) continue;
        if (!gated) epi_store<true>(e, b, j, acc[i]);
        else if ((lane & 1) == 0) epi_store_gated(e, b, j >> 1, acc[i], other);
    }
}

static const size_t kXLdsLimit = 48 * 1024;

// Waves per workgroup of the quantised decode matmul: enough waves to cover the chip several
// times over, at least 2 chunks per wave.
static uint32_t gemv_quant_waves(const Weight &w) {
    const uint32_t ngroups = (uint32_t)(w.k_pad / 128), tiles = (uint32_t)(w.n_pad / 16);
    uint32_t waves = 4;
    while (waves < 16 && (uint64_t)tiles * waves < 4096 && ngroups >= waves * 4) waves *= 2;
    while (waves > 1 && waves > ngroups) waves /= 2;
    return waves;
}

bool gemv_can_fuse_norm(const Weight &w, uint64_t batch) {
    if (w.dtype < COEUS_W_Q8_0 || batch < 1 || batch > 16) return false;
    const uint64_t bp = pad_batch(batch);
    return bp <= 4 && w.k_pad * bp * 2 <= kXLdsLimit &&
           w.k_pad / 8 * bp <= (uint64_t)NORM_PPT * gemv_quant_waves(w) * 64;
}

template <bool Q4, int BPV>
static void launch_gemv_quant_bp(int xmode, dim3 grid, dim3 block, size_t lds, hipStream_t st,
                                 const uint4 *qs, const uint2 *ds, const XArgs &xa,
                                 uint32_t ngroups, uint32_t b, const EpiArgs &e) {
    switch (xmode) {
        case X_GLOBAL:
            hipLaunchKernelGGL((gemv_quant_kernel<Q4, BPV, X_GLOBAL>), grid, block, lds, st, qs, ds, xa, ngroups, b, e);
            break;
        case X_LDS:
            hipLaunchKernelGGL((gemv_quant_kernel<Q4, BPV, X_LDS>), grid, block, lds, st, qs, ds, xa, ngroups, b, e);
            break;
        case X_LAYERNORM:
            if constexpr (BPV <= 4)
                hipLaunchKernelGGL((gemv_quant_kernel<Q4, BPV, X_LAYERNORM>), grid, block, lds, st, qs, ds, xa, ngroups, b, e);
            break;
        default:
            if constexpr (BPV <= 4)
                hipLaunchKernelGGL((gemv_quant_kernel<Q4, BPV, X_RMSNORM>), grid, block, lds, st, qs, ds, xa, ngroups, b, e);
            break;
    }
}

template <bool Q4>
static int launch_gemv_quant(const Weight &w, const __half *xq, uint64_t batch, const EpiArgs &e,
                             hipStream_t st, const NormFuse *nf) {
    const uint32_t ngroups = (uint32_t)(w.k_pad / 128), tiles = (uint32_t)(w.n_pad / 16);
    const uint32_t bp = pad_batch(batch), b = (uint32_t)batch;
    const uint32_t waves = gemv_quant_waves(w);
    const size_t x_bytes = (size_t)w.k_pad * bp * 2;
    const bool xlds = x_bytes <= kXLdsLimit;
    if (nf && !gemv_can_fuse_norm(w, batch))
        return fail(COEUS_INVALID_INPUT, "norm fusion needs the activations to fit in LDS");
    int xmode = xlds ? X_LDS : X_GLOBAL;
    XArgs xa{};
    xa.xq = (const uint4 *)xq;
    xa.k = (uint32_t)w.k;
    if (nf) {
        xmode = nf->kind == COEUS_NORM_RMSNORM ? X_RMSNORM : X_LAYERNORM;
        xa.h = nf->h; xa.nscale = nf->scale; xa.nbias = nf->bias; xa.eps = nf->eps;
    }
    const uint32_t ni = bp < 4 ? bp : 4;
    size_t red_bytes = waves > 1 ? (size_t)waves * ni * 64 * 4 : 0;
    if (nf && red_bytes < (size_t)waves * bp * 4) red_bytes = (size_t)waves * bp * 4;
    const size_t lds = (xlds ? x_bytes : 0) + red_bytes;
    const dim3 grid(tiles), block(waves * 64);
    const uint4 *qs = (const uint4 *)w.data;
    const uint2 *ds = (const uint2 *)w.scales;
    switch (bp) {
        case 1: launch_gemv_quant_bp<Q4, 1>(xmode, grid, block, lds, st, qs, ds, xa, ngroups, b, e); break;
        case 2: launch_gemv_quant_bp<Q4, 2>(xmode, grid, block, lds, st, qs, ds, xa, ngroups, b, e); break;
        case 4: launch_gemv_quant_bp<Q4, 4>(xmode, grid, block, lds, st, qs, ds, xa, ngroups, b, e); break;
        case 8: launch_gemv_quant_bp<Q4, 8>(xmode, grid, block, lds, st, qs, ds, xa, ngroups, b, e); break;
        default: launch_gemv_quant_bp<Q4, 16>(xmode, grid, block, lds, st, qs, ds, xa, ngroups, b, e); break;
    }
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

// ---------------------------------------------------------------- dense kernel (f32 / bf16)
template <bool BF16, int BP>
__global__ __launch_bounds__(256) void gemv_dense_kernel(const void *__restrict__ wdata,
                                                         const float *__restrict__ x, uint64_t k,
                                                         uint32_t batch, EpiArgs e) {
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint64_t j = (uint64_t)blockIdx.x * 4 + wave;
    if (j >= e.n) return;
    float acc[BP];
#pragma unroll
    for (int b = 0; b < BP; b++) acc[b] = 0.f;
    if ((k & 7) == 0) {
        for (uint64_t k0 = (uint64_t)lane * 8; k0 < k; k0 += 512) {
            float wv[8];
            if (BF16) {
                const uint4 raw = *(const uint4 *)((const uint16_t *)wdata + j * k + k0);
                const uint32_t r[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    wv[2 * t] = __uint_as_float(r[t] << 16);
                    wv[2 * t + 1] = __uint_as_float(r[t] & 0xffff0000u);
                }
            } else {
                const float4 a = *(const float4 *)((const float *)wdata + j * k + k0);
                const float4 b = *(const float4 *)((const float *)wdata + j * k + k0 + 4);
                wv[0] = a.x; wv[1] = a.y; wv[2] = a.z; wv[3] = a.w;
                wv[4] = b.x; wv[5] = b.y; wv[6] = b.z; wv[7] = b.w;
            }
#pragma unroll
            for (int b = 0; b < BP; b++) {
                if (b < (int)batch) {
                    const float4 xa = *(const float4 *)(x + (uint64_t)b * k + k0);
                    const float4 xb = *(const float4 *)(x + (uint64_t)b * k + k0 + 4);
                    float s = acc[b];
                    s = fmaf(wv[0], xa.x, s); s = fmaf(wv[1], xa.y, s);
                    s = fmaf(wv[2], xa.z, s); s = fmaf(wv[3], xa.w, s);
                    s = fmaf(wv[4], xb.x, s); s = fmaf(wv[5], xb.y, s);
                    s = fmaf(wv[6], xb.z, s); s = fmaf(wv[7], xb.w, s);
                    acc[b] = s;
                }
            }
        }
    } else {
        for (uint64_t kk = lane; kk < k; kk += 64) {
            const float wv = BF16 ? bf16_bits_to_f32(((const uint16_t *)wdata)[j * k + kk])
                                  : ((const float *)wdata)[j * k + kk];
#pragma unroll
            for (int b = 0; b < BP; b++)
                if (b < (int)batch) acc[b] = fmaf(wv, x[(uint64_t)b * k + kk], acc[b]);
        }
    }
#pragma unroll
    for (int b = 0; b < BP; b++) acc[b] = wave_sum(acc[b]);
    if (e.act == COEUS_EPI_SILU_GATE) {
        // pair (gate_m, up_m) = rows (2m, 2m+1) live in neighbouring waves: go through LDS
        __shared__ float pair[4][16];
        if (lane == 0)
#pragma unroll
            for (int b = 0; b < BP; b++) pair[wave][b] = acc[b];
        __syncthreads();
        if ((wave & 1) == 0 && lane < batch && j + 1 < e.n)
            epi_store_gated(e, lane, j / 2, pair[wave][lane], pair[wave + 1][lane]);
        return;
    }
    if (lane == 0)
#pragma unroll
        for (int b = 0; b < BP; b++)
            if (b < (int)batch) epi_store<true>(e, b, j, acc[b]);
}

template <bool BF16>
static int launch_gemv_dense(const Weight &w, const float *x, uint64_t batch, const EpiArgs &e,
                             hipStream_t st) {
    const dim3 grid((unsigned)ceil_div(w.n, 4)), block(256);
    const uint32_t bp = pad_batch(batch), b = (uint32_t)batch;
#define COEUS_GEMVD(BPV) \
    hipLaunchKernelGGL((gemv_dense_kernel<BF16, BPV>), grid, block, 0, st, w.data, x, w.k, b, e)
    switch (bp) {
        case 1: COEUS_GEMVD(1); break;
        case 2: COEUS_GEMVD(2); break;
        case 4: COEUS_GEMVD(4); break;
        case 8: COEUS_GEMVD(8); break;
        default: COEUS_GEMVD(16); break;
    }
#undef COEUS_GEMVD
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

int launch_gemv(const Weight &w, const void *x, uint64_t batch, const Epilogue &ep, hipStream_t st,
                const NormFuse *nf) {
    if (batch == 0 || batch > 16)
        return fail(COEUS_INVALID_INPUT, "decode matmul batch %llu out of range [1, 16]",
                    (unsigned long long)batch);
    if (ep.act == COEUS_EPI_SILU_GATE && (w.n & 1))
        return fail(COEUS_INVALID_INPUT, "gated epilogue needs an even number of weight rows");
    const EpiArgs e = make_epi(ep, w.n);
    if (nf && w.dtype < COEUS_W_Q8_0)
        return fail(COEUS_INVALID_INPUT, "norm fusion is implemented for quantised weights only");
    switch (w.dtype) {
        case COEUS_W_F32: return launch_gemv_dense<false>(w, (const float *)x, batch, e, st);
        case COEUS_W_BF16: return launch_gemv_dense<true>(w, (const float *)x, batch, e, st);
        case COEUS_W_Q8_0: return launch_gemv_quant<false>(w, (const __half *)x, batch, e, st, nf);
        default: return launch_gemv_quant<true>(w, (const __half *)x, batch, e, st, nf);
    }
}

}  // namespace coeus
