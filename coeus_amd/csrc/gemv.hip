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

template <bool Q4, int BP, bool XLDS>
__global__ __launch_bounds__(1024) void gemv_quant_kernel(const uint4 *__restrict__ qs,
                                                          const uint2 *__restrict__ ds,
                                                          const uint4 *__restrict__ xq,
                                                          uint32_t ngroups, uint32_t batch,
                                                          EpiArgs e) {
    constexpr int NI = BP < 4 ? BP : 4;  // accumulator rows that can hold a real batch entry
    extern __shared__ uint4 smem[];      // [x: ngroups*16*BP uint4 if XLDS][reduction]
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    const uint32_t T = blockIdx.x;
    const uint32_t g = lane >> 4, xb = (lane & 15) & (BP - 1);
    float acc[NI];
#pragma unroll
    for (int i = 0; i < NI; i++) acc[i] = 0.f;
    const float4_t zero = {0.f, 0.f, 0.f, 0.f};

    // PF chunks (PF KiB of Q4_0 quants per wave) are requested before any of them is used:
    // with ~24 waves per CU that keeps enough bytes in flight to cover HBM latency.
    constexpr int PF = 4;
    const uint32_t nx = ngroups * 16 * BP;  // uint4 pieces of the activation block
    bool staged = !XLDS;
    for (uint32_t G0 = wave; G0 < ngroups; G0 += nwaves * PF) {
        ChunkRegs<Q4> r[PF];
#pragma unroll
        for (int u = 0; u < PF; u++) {
            const uint32_t G = G0 + u * nwaves;
            if (G < ngroups) load_chunk<Q4>(r[u], qs, ds, (uint64_t)T * ngroups + G, lane);
        }
        if (!staged) {  // first pass only; uniform across the workgroup
            for (uint32_t i = threadIdx.x; i < nx; i += blockDim.x) smem[i] = xq[i];
            __syncthreads();
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
                union { uint4 u4; half8_t h; } xa;
                xa.u4 = XLDS ? smem[xi] : xq[xi];
                const half8_t wv = Q4 ? unpack_q4(qw[jj]) : unpack_q8(qw[2 * jj], qw[2 * jj + 1]);
                const float4_t part = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa.h, wv, zero, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < NI; i++) acc[i] = fmaf(d[jj], part[i], acc[i]);
            }
        }
    }
    if (!staged) {  // a wave without chunks still takes part in the staging
        for (uint32_t i = threadIdx.x; i < nx; i += blockDim.x) smem[i] = xq[i];
        __syncthreads();
    }

    // deterministic cross-wave reduction (fixed order), then the epilogue on wave 0
    if (nwaves > 1) {
        float *red = (float *)(smem + (XLDS ? nx : 0));
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
        if (!gated) epi_store(e, b, j, acc[i]);
        else if ((lane & 1) == 0) epi_store_gated(e, b, j >> 1, acc[i], other);
    }
}

template <bool Q4>
static int launch_gemv_quant(const Weight &w, const __half *xq, uint64_t batch, const EpiArgs &e,
                             hipStream_t st) {
    const uint32_t ngroups = (uint32_t)(w.k_pad / 128), tiles = (uint32_t)(w.n_pad / 16);
    const uint32_t bp = pad_batch(batch), b = (uint32_t)batch;
    // enough waves to cover the chip several times over, at least 2 chunks per wave
    uint32_t waves = 4;
    while (waves < 16 && (uint64_t)tiles * waves < 4096 && ngroups >= waves * 4) waves *= 2;
    while (waves > 1 && waves > ngroups) waves /= 2;
    const size_t x_bytes = (size_t)w.k_pad * bp * 2;
    const bool xlds = x_bytes <= 48 * 1024;
    const uint32_t ni = bp < 4 ? bp : 4;
    const size_t lds = (xlds ? x_bytes : 0) + (waves > 1 ? (size_t)waves * ni * 64 * 4 : 0);
    const dim3 grid(tiles), block(waves * 64);
    const uint4 *qs = (const uint4 *)w.data, *x4 = (const uint4 *)xq;
    const uint2 *ds = (const uint2 *)w.scales;
#define COEUS_GEMVQ(BPV)                                                                          \
    do {                                                                                          \
        if (xlds)                                                                                 \
            hipLaunchKernelGGL((gemv_quant_kernel<Q4, BPV, true>), grid, block, lds, st, qs, ds,  \
                               x4, ngroups, b, e);                                                \
        else                                                                                      \
            hipLaunchKernelGGL((gemv_quant_kernel<Q4, BPV, false>), grid, block, lds, st, qs, ds, \
                               x4, ngroups, b, e);                                                \
    } while (0)
    switch (bp) {
        case 1: COEUS_GEMVQ(1); break;
        case 2: COEUS_GEMVQ(2); break;
        case 4: COEUS_GEMVQ(4); break;
        case 8: COEUS_GEMVQ(8); break;
        default: COEUS_GEMVQ(16); break;
    }
#undef COEUS_GEMVQ
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
            if (b < (int)batch) epi_store(e, b, j, acc[b]);
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

int launch_gemv(const Weight &w, const void *x, uint64_t batch, const Epilogue &ep, hipStream_t st) {
    if (batch == 0 || batch > 16)
        return fail(COEUS_INVALID_INPUT, "decode matmul batch %llu out of range [1, 16]",
                    (unsigned long long)batch);
    if (ep.act == COEUS_EPI_SILU_GATE && (w.n & 1))
        return fail(COEUS_INVALID_INPUT, "gated epilogue needs an even number of weight rows");
    const EpiArgs e = make_epi(ep, w.n);
    switch (w.dtype) {
        case COEUS_W_F32: return launch_gemv_dense<false>(w, (const float *)x, batch, e, st);
        case COEUS_W_BF16: return launch_gemv_dense<true>(w, (const float *)x, batch, e, st);
        case COEUS_W_Q8_0: return launch_gemv_quant<false>(w, (const __half *)x, batch, e, st);
        default: return launch_gemv_quant<true>(w, (const __half *)x, batch, e, st);
    }
}

}  // namespace coeus
