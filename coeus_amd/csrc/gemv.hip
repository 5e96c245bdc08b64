// Decode matmul: y[b, :] = x[b, :] . W for b < batch <= 16 (math::matmul, MT:50-74, with
// m = batch), the HBM-bound kernel of token generation.
//
//   gemv_quad_kernel   Q8_0 / Q4_0 weights in MFMA-native tiles, batches of up to 4 (the kernel of
//                      single-sequence generation): one workgroup per tile of 16 output rows, a
//                      wave owns four consecutive 128-k chunks, stages exactly their activations
//                      (with or without the folded norm) into its private slice of LDS and feeds
//                      the quants to v_mfma_f32_16x16x32_f16 as f16 subnormals.
//   gemv_quant_kernel  the same weights for batches of 5 to 16.  One workgroup owns a tile of
//                      16 output rows (or four); its waves take interleaved 128-k chunks (1 KiB
//                      of Q4_0 quants = one fully coalesced 16 B/lane load per wave).  Each 32-k
//                      block is one v_mfma_f32_16x16x32_f16 between the 16 activation rows (f16)
//                      and the block's integers (q-8 resp. q, exact in f16); the f32 block result
//                      is scaled by the block's f16 scale on the VALU.  Activation rows come from
//                      LDS (staged once per workgroup) or, when they do not fit, from L2 product
//                      by product; there a workgroup takes four tiles and a wave multiplies each
//                      fragment with all four.  In both kernels the value used for every weight is
//                      exactly its dequantised value q*d.
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
    // (the scales are read once per step like the quants: 1.753 -> 1.722 ms per 7B batch-1 step with
    // this load non-temporal too)
    typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
    const u32x2_t sv = __builtin_nontemporal_load((const u32x2_t *)(ds + chunk * 16 + (lane & 15)));
    r.s = make_uint2(sv.x, sv.y);
}

// How the activation block reaches the matrix cores.
enum { X_GLOBAL = 0,  // xq read from global memory (L2) per block: no LDS needed, any size (gemv_quant_kernel)
       X_LDS = 1,     // xq copied into LDS (once per workgroup; gemv_quad_kernel: each wave its own pieces)
       X_LAYERNORM = 2, X_RMSNORM = 3,    // gemv_quad_kernel: f32 residual rows normalised while staged into LDS
       X_RMSPRE = 4 };  // gemv_quad_kernel: rows that their producer stored as h * scale: times 1 / rms while staged

struct XArgs {
    const uint4 *xq;      // X_GLOBAL / X_LDS
    const float *h;       // X_*NORM: [batch, k]; X_RMSPRE: the rows times the norm's scale
    const float *nscale, *nbias;
    const float2 *stats;  // X_*NORM: [batch][ceil(k/16)] {sum, M2} records of h
    float eps;
    uint32_t k;           // logical reduction length
};

// The same normalisation as a launch of its own, for batches whose activation block does not fit
// the matmul's LDS staging: row b of h -> xq, statistics merged from the producer's records
// (no reduction over the row).  Grid (k pieces / 256, batch); every wave merges its row's records.
template <bool RMS>
__global__ __launch_bounds__(256) void norm_from_stats_kernel(const float *__restrict__ h,
                                                              const float2 *__restrict__ stats,
                                                              const float *__restrict__ nscale,
                                                              const float *__restrict__ nbias,
                                                              float eps, uint32_t k, uint32_t k_pad,
                                                              uint32_t bp, uint4 *__restrict__ xq) {
    const uint32_t lane = threadIdx.x & 63, b = blockIdx.y, nt = (k + 15) / 16;
    const uint32_t kp = blockIdx.x * 256 + threadIdx.x;  // piece = 8 consecutive k
    const float2 *rec = stats + (uint64_t)b * nt;
    float s = 0.f;
    for (uint32_t t = lane; t < nt; t += 64) s += rec[t].x;
    const float rk = __builtin_amdgcn_rcpf((float)k);
    const float mean = RMS ? 0.f : wave_sum(s) * rk;
    const uint32_t tail = k & 15;
    float q = 0.f;
    for (uint32_t t = lane; t < nt; t += 64) {
        const bool last = tail && t == nt - 1;
        const float c = last ? (float)tail : 16.f;
        const float d = rec[t].x * __builtin_amdgcn_rcpf(c) - mean;
        q += fmaf(c * d, d, rec[t].y);
    }
    const float rsd = __builtin_amdgcn_rsqf(wave_sum(q) * rk + eps);
    if (kp >= k_pad / 8) return;
    uint4 o = make_uint4(0, 0, 0, 0);
    const uint32_t kk = kp * 8;
    if (kk < k) {  // k % 8 == 0
        const float4 a0 = *(const float4 *)(h + (uint64_t)b * k + kk), a1 = *(const float4 *)(h + (uint64_t)b * k + kk + 4);
        const float4 s0 = *(const float4 *)(nscale + kk), s1 = *(const float4 *)(nscale + kk + 4);
        const float v[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
        const float sc[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
        float y[8];
#pragma unroll
        for (int u = 0; u < 8; u++) y[u] = (v[u] - mean) * (sc[u] * rsd);
        if (!RMS) {
            const float4 b0 = *(const float4 *)(nbias + kk), b1 = *(const float4 *)(nbias + kk + 4);
            const float bi[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
#pragma unroll
            for (int u = 0; u < 8; u++) y[u] += bi[u];
        }
        union { uint4 u; half2_t h2[4]; } cv;
#pragma unroll
        for (int u = 0; u < 4; u++) {
            cv.h2[u].x = (_Float16)y[2 * u];
            cv.h2[u].y = (_Float16)y[2 * u + 1];
        }
        o = cv.u;
    }
    xq[(uint64_t)kp * bp + b] = o;
}

int launch_norm_from_stats(const NormFuse &nf, uint64_t batch, uint64_t k, uint64_t k_pad, __half *xq,
                           hipStream_t st) {
    if (!nf.stats || (k & 7))
        return fail(COEUS_INVALID_INPUT, "norm from statistics needs the records and k %% 8 == 0");
    const uint32_t bp = pad_batch(batch);
    const dim3 grid((unsigned)ceil_div(k_pad / 8, 256), (unsigned)batch);
    if (nf.kind == COEUS_NORM_RMSNORM)
        hipLaunchKernelGGL(norm_from_stats_kernel<true>, grid, dim3(256), 0, st, nf.h, nf.stats, nf.scale, nf.bias, nf.eps, (uint32_t)k, (uint32_t)k_pad, bp, (uint4 *)xq);
    else
        hipLaunchKernelGGL(norm_from_stats_kernel<false>, grid, dim3(256), 0, st, nf.h, nf.stats, nf.scale, nf.bias, nf.eps, (uint32_t)k, (uint32_t)k_pad, bp, (uint4 *)xq);
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

// Compile-time shape of one gemv_quant_kernel variant, packed into an int:
//   bit 0     always set
//   bit 5     two tiles per workgroup
//   bit 6     6 chunks in flight per wave instead of 4 (Q8_0: 3 instead of 2)
//   bit 7     2 chunks in flight per wave instead of 4 (Q8_0: 1): short reductions, where the waves
//             of a workgroup cover k in fewer chunks and the extra requests would be re-reads
//   bit 8     four tiles per workgroup (activations from global memory only)
constexpr int CFG_TPW2 = 32, CFG_PF6 = 64, CFG_PF2 = 128, CFG_TPW4 = 256;

// One workgroup takes TPW tiles of 16 output rows; several workgroups share a CU, so that the
// staging and the epilogue of one overlap with the weight stream of the others (the register
// budget is capped to keep 6-8 waves per SIMD resident).  With TPW = 2 the activation block is
// staged once for two tiles and both tiles' chunks are requested before either is used.
// Activations that do not fit LDS are read from global memory (L2) product by product; there a
// wave takes its chunks of all TPW tiles (2 or 4), so that one activation fragment (1 KiB per
// product at 16 batch rows, against 288 bytes of Q4_0 weights) serves TPW products.
template <bool Q4, int BP, int XMODE, int CFG>
__global__ __launch_bounds__(1024)
__attribute__((amdgpu_waves_per_eu((XMODE == X_GLOBAL && (CFG & (CFG_TPW2 | CFG_TPW4))) ? 4 : 6, 8)))
void gemv_quant_kernel(const uint4 *__restrict__ qs, const uint2 *__restrict__ ds, XArgs xa,
                       uint32_t ngroups, uint32_t tiles, uint32_t batch, EpiArgs e) {
    static_assert(BP == 8 || BP == 16, "batches of up to 4 take gemv_quad_kernel");
    static_assert(XMODE == X_GLOBAL || XMODE == X_LDS, "activations from L2 or staged in LDS");
    constexpr int NI = 4;  // accumulator rows of a lane
    constexpr bool XLDS = XMODE != X_GLOBAL;
    constexpr int TPW = (CFG & CFG_TPW4) ? 4 : (CFG & CFG_TPW2) ? 2 : 1;
    constexpr bool SHARE_X = XMODE == X_GLOBAL && TPW > 1;
    extern __shared__ uint4 smem[];      // [x: ngroups*16*BP uint4 if XLDS][reduction]
    const uint32_t lane = threadIdx.x & 63, nwaves = blockDim.x >> 6;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t T0 = blockIdx.x * TPW;
    const uint32_t g = lane >> 4, xb = (lane & 15) & (BP - 1);
    float acc[NI];
#pragma unroll
    for (int i = 0; i < NI; i++) acc[i] = 0.f;
    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
    const uint4 *__restrict__ xq = xa.xq;
    const uint32_t nx = ngroups * 16 * BP;  // uint4 pieces of the activation block
    float *red = (float *)(smem + (XLDS ? nx : 0));  // [TPW][nwaves][NI][64]

    // 0. the residual elements this wave will need if it runs a tile's epilogue (wave t < TPW
    // finishes tile T0 + t): requested now, unconditionally (other waves repeat wave 0's, a
    // missing residual reads a valid dummy), so the epilogue does not wait for a load of its own
    constexpr bool RES_PRE = true;
    float res_pre[NI];
    {
        const float *rp = e.residual ? e.residual : (const float *)ds;
        const uint32_t Tw = min(T0 + (wave < (uint32_t)TPW ? wave : 0u), tiles - 1);
        const uint64_t jp = (uint64_t)Tw * 16 + (lane & 15);
#pragma unroll
        for (int i = 0; i < NI; i++) {
            const uint32_t b = 4 * g + i;
            const bool ok = e.residual && b < batch && jp < e.n;
            res_pre[i] = rp[ok ? (uint64_t)b * e.n_eff + jp : 0];
        }
    }

    // 1. activations first: a wave's loads are answered in order, and these are needed first
    constexpr int XPT = 2;
    uint4 xr[XPT];
    if (XMODE == X_LDS) {
#pragma unroll
        for (int u = 0; u < XPT; u++) {
            const uint32_t i = threadIdx.x + u * blockDim.x;
            xr[u] = xq[i < nx ? i : 0];  // unconditional, from a clamped address (see step 2)
        }
    }
    auto stage = [&]() {
        if (XMODE == X_LDS) {
#pragma unroll
            for (int u = 0; u < XPT; u++) {
                const uint32_t i = threadIdx.x + u * blockDim.x;
                if (i < nx) smem[i] = xr[u];
            }
            for (uint32_t i = threadIdx.x + XPT * blockDim.x; i < nx; i += blockDim.x) smem[i] = xq[i];
        }
        if (XLDS) lds_barrier();
    };

    // 2. PF chunks (PF KiB of Q4_0 quants per wave and tile) are requested before any of them is
    // used.  Passes in which every wave has all its chunks use unconditional loads: the compiler
    // then knows exactly how many loads are in flight, and the staging and the first chunks are
    // used while later ones are still on their way.  (A load under a branch makes it wait for
    // everything.)  Only a last partial pass loads under wave-uniform branches.
    constexpr int PF = (CFG & CFG_PF6) ? (Q4 ? 6 : 3) : (CFG & CFG_PF2) ? (Q4 ? 2 : 1) : (Q4 ? 4 : 2);
    auto consume = [&](const ChunkRegs<Q4> &r, uint32_t G) {
        const uint32_t qw[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, Q4 ? 0u : r.q1.x, Q4 ? 0u : r.q1.y,
                                Q4 ? 0u : r.q1.z, Q4 ? 0u : r.q1.w};
        union { uint2 u2; half2_t h[2]; } sc;
        sc.u2 = r.s;
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
    };
    // a tile's partial result of this wave, parked for the cross-wave sum
    auto park = [&](int t) {
#pragma unroll
        for (int i = 0; i < NI; i++) {
            red[((t * nwaves + wave) * NI + i) * 64 + lane] = acc[i];
            acc[i] = 0.f;
        }
    };
    if constexpr (SHARE_X) {
        // a wave's chunk G of every tile, against one set of activation fragments
        constexpr int PFS = (!Q4 && TPW == 4) ? 1 : 2;  // chunks of a tile in flight per wave
        float accs[TPW][NI];
        uint64_t cb[TPW];
#pragma unroll
        for (int t = 0; t < TPW; t++) {
            cb[t] = (uint64_t)min(T0 + t, tiles - 1) * ngroups;
#pragma unroll
            for (int i = 0; i < NI; i++) accs[t][i] = 0.f;
        }
        auto pass = [&](uint32_t Gp, auto full) {
            ChunkRegs<Q4> r[PFS][TPW];
            uint4 xv[PFS][4];
#pragma unroll
            for (int u = 0; u < PFS; u++) {
                const uint32_t G = Gp + u * nwaves;
                if (decltype(full)::value || G < ngroups) {
#pragma unroll
                    for (int jj = 0; jj < 4; jj++) xv[u][jj] = xq[((G * 4 + jj) * 4 + g) * BP + xb];
#pragma unroll
                    for (int t = 0; t < TPW; t++) load_chunk<Q4>(r[u][t], qs, ds, cb[t] + G, lane);
                }
            }
#pragma unroll
            for (int u = 0; u < PFS; u++) {
                if (decltype(full)::value || Gp + u * nwaves < ngroups) {
#pragma unroll
                    for (int t = 0; t < TPW; t++) {
                        const ChunkRegs<Q4> &c = r[u][t];
                        const uint32_t qw[8] = {c.q0.x, c.q0.y, c.q0.z, c.q0.w, Q4 ? 0u : c.q1.x, Q4 ? 0u : c.q1.y,
                                                Q4 ? 0u : c.q1.z, Q4 ? 0u : c.q1.w};
                        union { uint2 u2; half2_t h[2]; } sc;
                        sc.u2 = c.s;
                        const float d[4] = {(float)sc.h[0].x, (float)sc.h[0].y, (float)sc.h[1].x, (float)sc.h[1].y};
#pragma unroll
                        for (int jj = 0; jj < 4; jj++) {
                            union { uint4 u4; half8_t h; } xf;
                            xf.u4 = xv[u][jj];
                            const half8_t wv = Q4 ? unpack_q4(qw[jj]) : unpack_q8(qw[2 * jj], qw[2 * jj + 1]);
                            const float4_t part = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf.h, wv, zero, 0, 0, 0);
#pragma unroll
                            for (int i = 0; i < NI; i++) accs[t][i] = fmaf(d[jj], part[i], accs[t][i]);
                        }
                    }
                }
            }
        };
        uint32_t Gp = wave;
        for (; Gp + (PFS - 1) * nwaves < ngroups; Gp += nwaves * PFS) pass(Gp, std::true_type{});
        if (Gp < ngroups) pass(Gp, std::false_type{});
#pragma unroll
        for (int t = 0; t < TPW; t++)
#pragma unroll
            for (int i = 0; i < NI; i++) red[((t * nwaves + wave) * NI + i) * 64 + lane] = accs[t][i];
    } else {
        uint32_t G0 = wave;  // < ngroups: a workgroup never has more waves than chunks
        {   // first pass, always with unconditional loads (a slot past the end re-reads a valid
            // chunk and is not used)
            ChunkRegs<Q4> r[TPW][PF];
    #pragma unroll
            for (int t = 0; t < TPW; t++) {
                const uint64_t cbase = (uint64_t)min(T0 + t, tiles - 1) * ngroups;
    #pragma unroll
                for (int u = 0; u < PF; u++)
                    load_chunk<Q4>(r[t][u], qs, ds, cbase + min(G0 + u * nwaves, ngroups - 1), lane);
            }
            stage();
    #pragma unroll
            for (int t = 0; t < TPW; t++) {
    #pragma unroll
                for (int u = 0; u < PF; u++)
                    if (G0 + u * nwaves < ngroups) consume(r[t][u], G0 + u * nwaves);
                if (TPW > 1) park(t);  // two tiles per workgroup: the reduction takes a single pass
            }
        }
        if (TPW == 1) {
            const uint64_t cbase = (uint64_t)T0 * ngroups;
            for (G0 += nwaves * PF; G0 + (PF - 1) * nwaves < ngroups; G0 += nwaves * PF) {
                ChunkRegs<Q4> r[PF];
    #pragma unroll
                for (int u = 0; u < PF; u++) load_chunk<Q4>(r[u], qs, ds, cbase + G0 + u * nwaves, lane);
    #pragma unroll
                for (int u = 0; u < PF; u++) consume(r[u], G0 + u * nwaves);
            }
            if (G0 < ngroups) {  // partial last pass
                ChunkRegs<Q4> r[PF];
    #pragma unroll
                for (int u = 0; u < PF; u++)
                    if (G0 + u * nwaves < ngroups) load_chunk<Q4>(r[u], qs, ds, cbase + G0 + u * nwaves, lane);
    #pragma unroll
                for (int u = 0; u < PF; u++)
                    if (G0 + u * nwaves < ngroups) consume(r[u], G0 + u * nwaves);
            }
        }

    }

    // deterministic cross-wave reduction (fixed order); wave t runs the epilogue of tile T0 + t
    uint32_t T = T0;
    if (nwaves > 1 || TPW > 1) {
        if (TPW == 1) park(0);  // (several tiles: parked above)
        lds_barrier();
        if (wave >= (uint32_t)TPW) return;
        T = T0 + wave;
        if (T >= tiles) return;
        for (uint32_t w = 0; w < nwaves; w++)
#pragma unroll
            for (int i = 0; i < NI; i++) acc[i] += red[((wave * nwaves + w) * NI + i) * 64 + lane];
    }
    const uint64_t j = (uint64_t)T * 16 + (lane & 15);
    const bool gated = e.act == COEUS_EPI_SILU_GATE;
#pragma unroll
    for (int i = 0; i < NI; i++) {
        const uint32_t b = 4 * g + i;
        // gated: weight rows (2m, 2m+1) = (gate_m, up_m) sit in neighbouring lanes
        const float other = lane_xor1(acc[i]);
        const bool live = b < batch && j < e.n;
        float v = 0.f;
        if (live) {
            if (!gated) v = epi_store<true>(e, b, j, acc[i], RES_PRE, res_pre[i]);
            else if ((lane & 1) == 0) epi_store_gated(e, b, j >> 1, acc[i], other);
        }
        if (e.stats_out) {  // uniform; never combined with the gated epilogue
            const uint32_t left = (uint32_t)e.n - T * 16;
            const float2 r = group16_stats(v, live, left < 16 ? left : 16u);
            if ((lane & 15) == 0 && b < batch) e.stats_out[(uint64_t)b * e.stats_tiles + T] = r;
        }
    }
}

// ---------------------------------------------------------------- quad kernel (batches of up to 4)
// The decode matmul for batch <= 4, where a launch is a transient: the whole matrix (10-70 MB) is
// requested within the first microsecond and the kernel ends when the last line has arrived, so
// what counts is that every wave asks for its weights at once, that as few other bytes as possible
// go through the CU's memory pipeline, and that little is left to do after the last line.  A wave
// owns "quads" of four consecutive 128-k chunks of its workgroup's tile (4 KiB of Q4_0 quants per
// quad) and does everything for them on its own:
//   * it requests, in this order, the activations of exactly its quads (or, with a folded norm,
//     the residual values, scale and bias of those k; the row's statistics records are read by
//     wave 0 alone), the block scales (ONE 8-byte load per lane for a whole quad: lane 16 u + r takes
//     the four scales of row r in chunk u), then the quants; all unconditional, from clamped
//     addresses;
//   * as soon as the activation loads have arrived (the weights are still in flight) it
//     normalises / copies them into its PRIVATE slice of LDS as f16 matrix-core fragments; no
//     workgroup barrier orders this (the one barrier of a folded norm hands out the row statistics):
//     a wave only ever reads fragments that it wrote itself;
//   * the quants enter the matrix cores as they are stored: a masked nibble (or a byte) IS the bit
//     pattern of the f16 subnormal n * 2^-24, which v_mfma_f32_16x16x32_f16 multiplies exactly, so
//     a 32-k block costs one shift and four ANDs instead of the conversion to q - 8.  Nibbles kept
//     at bit 4 count 16-fold; the activations of those k positions are staged divided by 16.  The
//     offset comes back through the block's activation sum S: d * (sum x n - 8 S) = sum x (n - 8) d;
//   * chunk u of a quad is multiplied by all 64 lanes (activations replicated over the 16 A rows by
//     row % BP), but only the lanes 16 u .. 16 u + 15 add the scaled block result to their
//     accumulators, because they are the ones that hold chunk u's scales; the four lane groups are
//     summed once at the end.
// The waves' partial sums meet in LDS (16 floats per wave and batch row), and wave 0 adds them up
// and runs the epilogue with one output element per lane (lane = 16 b + column), on operands
// (residual element, cache position) that were requested at kernel start.
template <bool Q4>
__device__ __forceinline__ half8_t quad_operand(uint32_t w0, uint32_t w1) {
    union { uint32_t u[4]; half8_t h; } o;
    if (Q4) {  // nibble positions [k0,k2,k4,k6,k1,k3,k5,k7]: (k0,k1) (k2,k3)<<4 (k4,k5) (k6,k7)<<4
        const uint32_t w8 = w0 >> 8;
        o.u[0] = w0 & 0x000F000Fu; o.u[1] = w0 & 0x00F000F0u; o.u[2] = w8 & 0x000F000Fu; o.u[3] = w8 & 0x00F000F0u;
    } else {   // int8 -> q + 128 in the low byte of each half
        const uint32_t l = w0 ^ 0x80808080u, h = w1 ^ 0x80808080u;
        o.u[0] = __builtin_amdgcn_perm(0u, l, 0x0c010c00u); o.u[1] = __builtin_amdgcn_perm(0u, l, 0x0c030c02u);
        o.u[2] = __builtin_amdgcn_perm(0u, h, 0x0c010c00u); o.u[3] = __builtin_amdgcn_perm(0u, h, 0x0c030c02u);
    }
    return o.h;
}

// One staged piece: 8 consecutive k of one batch row as f16.  Returns what goes into LDS (Q4_0: the
// values that meet a nibble kept at bit 4 divided by 16, rounded to f16 once more, which only changes
// values below 2^-10, by at most 2^-21) and adds the piece's share of the block's activation sum.
template <bool Q4>
__device__ __forceinline__ uint4 quad_piece(uint4 piece, float &sum) {
    union { uint4 u; half2_t h2[4]; } o;
    o.u = piece;
    if (Q4) {
        const half2_t r16 = {(_Float16)0.0625f, (_Float16)0.0625f};
        o.h2[1] = o.h2[1] * r16;
        o.h2[3] = o.h2[3] * r16;
        sum = ((float)o.h2[0].x + (float)o.h2[0].y) + ((float)o.h2[2].x + (float)o.h2[2].y) +
              16.f * (((float)o.h2[1].x + (float)o.h2[1].y) + ((float)o.h2[3].x + (float)o.h2[3].y));
    } else {
        sum = ((float)o.h2[0].x + (float)o.h2[0].y) + ((float)o.h2[1].x + (float)o.h2[1].y) +
              ((float)o.h2[2].x + (float)o.h2[2].y) + ((float)o.h2[3].x + (float)o.h2[3].y);
    }
    return o.u;
}

template <bool Q4, int BP, int XMODE, int QPW, int SREC>
__global__ __launch_bounds__((BP == 4 && XMODE != X_LDS) ? 512 : 1024)  // (four rows with a folded norm: k <= 4096, 8 waves)
__attribute__((amdgpu_waves_per_eu((Q4 && BP * QPW == 1 && XMODE != X_LAYERNORM) ? 6 :
                                   (BP * QPW <= 2 || XMODE == X_LDS) ? 4 : 2, 8)))
void gemv_quad_kernel(const uint4 *__restrict__ qs, const uint2 *__restrict__ ds, XArgs xa, uint32_t ngroups,
                      uint32_t tiles, uint32_t batch, EpiArgs e) {
    static_assert(BP == 1 || BP == 2 || BP == 4, "batch padded to 1, 2 or 4");
    // NORM: f32 rows are normalised while staged; PRE: rows already multiplied by the scale (RMSNorm)
    constexpr bool PRE = XMODE == X_RMSPRE, NORM = XMODE == X_LAYERNORM || XMODE == X_RMSNORM || PRE;
    constexpr bool RMS = XMODE == X_RMSNORM || PRE;
    static_assert(!NORM || QPW == 1, "a folded norm stages one quad per wave");
    constexpr int NI = BP;
    constexpr int WSTRIDE = QPW * BP * 68;  // uint4 per wave: 64 pieces and 16 block sums per quad and batch row
    extern __shared__ uint4 smem[];         // [nwaves][WSTRIDE], partial sums [nwaves][NI][16], row statistics [BP]
    const uint32_t lane = threadIdx.x & 63, nwaves = blockDim.x >> 6;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t j = lane & 15, ig = lane >> 4;
    const uint32_t T = blockIdx.x, nquads = (ngroups + 3) / 4;
    uint4 *xw = smem + wave * WSTRIDE;
    float *sw = (float *)(xw + QPW * BP * 64);  // [QPW][16 blocks][BP]: -8 (or -128) * the block's activation sum
    float *red = (float *)(smem + nwaves * WSTRIDE);
    float2 *rowstat = (float2 *)(red + nwaves * NI * 16);  // {mean, 1 / standard deviation} per batch row

    const uint32_t k = xa.k, nt = (k + 15) / 16;
    // a folded norm: wave 0 also merges the producer's statistics records of the rows (requested first)
    float2 rec0[NORM ? BP : 1][NORM ? SREC : 1];
    if constexpr (NORM) {
        if (wave == 0) {
#pragma unroll
            for (int b = 0; b < BP; b++) {
                const uint32_t bc = (uint32_t)b < batch ? b : 0;
#pragma unroll
                for (int u = 0; u < SREC; u++) rec0[b][u] = xa.stats[(uint64_t)bc * nt + min(lane + 64 * u, nt - 1)];
            }
        }
    }

    // 0. What the epilogue needs is requested now, so that nothing at the end of the kernel waits for
    // a load of its own: the operands of lane (b = ig, column j), by every wave though only wave 0
    // uses them (a load under a branch would make the compiler wait for every request at once).
    float *out_f32 = e.out_f32;
    __half *out_xq = e.out_xq;
    uint16_t *out_lp = e.out_lp;
    float2 *stats_out = e.stats_out;
    void *kv_k = e.kv_k, *kv_v = e.kv_v;
    uint32_t ep_act = e.act, bp_out = e.bp_out, kv_dtype = e.kv_dtype, kv_inner = e.kv_inner, stats_tiles = e.stats_tiles,
             lp_ld = e.lp_ld, lp_bf16 = e.lp_bf16;
    uint64_t ep_n = e.n, n_eff = e.n_eff;
    const uint64_t col = (uint64_t)T * 16 + j;
    const bool gated = ep_act == COEUS_EPI_SILU_GATE;
    const uint32_t kvpos = e.kv_pos ? *e.kv_pos : 0u;
    float res_pre, bias_pre, gs_pre;
    {
        const float *gp = e.g_out ? e.g_scale : (const float *)ds;
        gs_pre = gp[(e.g_out && col < ep_n) ? col : 0];
        const float *rp = (e.residual && !gated) ? e.residual : (const float *)ds;
        const bool ok = e.residual && !gated && ig < batch && col < ep_n;
        res_pre = rp[ok ? (uint64_t)ig * n_eff + col : 0];
        res_pre = ok ? res_pre : 0.f;
        const float *bp = e.bias ? e.bias : (const float *)ds;
        bias_pre = bp[(e.bias && col < ep_n) ? col : 0];
        bias_pre = e.bias ? bias_pre : 0.f;
    }
    // q|k|v: a tile lies inside one head of one of the three parts when both sizes are multiples
    // of 16; where its 16 outputs go in the cache is worked out here, off the tail
    const bool kv_odd = kv_k && ((kv_inner | e.kv_hd) & 15u);
    const bool kv_tile = kv_k && !kv_odd && T * 16 >= kv_inner;
    uint64_t kv_idx = 0;

    float acc[NI];
#pragma unroll
    for (int i = 0; i < NI; i++) acc[i] = 0.f;
    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
    const uint64_t cb = (uint64_t)T * ngroups;

    for (uint32_t qb = 0; qb < nquads; qb += nwaves * QPW) {  // (a folded norm: exactly one pass)
        const uint32_t q0 = qb + wave * QPW;
        // ---- 1. activations of this wave's quads: lane (u = ig, piece j) of chunk 4 q + u
        uint4 xr[QPW][BP];
        float4 hv[NORM ? BP : 1][2], scv[2], biv[2];
        if constexpr (NORM) {
            const uint32_t G = 4 * q0 + ig;
            uint32_t kk = (G * 16 + j) * 8;
            kk = (G < ngroups && kk < k) ? kk : 0;  // k % 8 == 0: a piece is all in or all out
#pragma unroll
            for (int b = 0; b < BP; b++) {
                const uint32_t bc = (uint32_t)b < batch ? b : 0;
                hv[b][0] = *(const float4 *)(xa.h + (uint64_t)bc * k + kk);
                hv[b][1] = *(const float4 *)(xa.h + (uint64_t)bc * k + kk + 4);
            }
            if (!PRE) {
                scv[0] = *(const float4 *)(xa.nscale + kk);
                scv[1] = *(const float4 *)(xa.nscale + kk + 4);
            }
            if (!RMS) {
                biv[0] = *(const float4 *)(xa.nbias + kk);
                biv[1] = *(const float4 *)(xa.nbias + kk + 4);
            }
        } else {
#pragma unroll
            for (int s = 0; s < QPW; s++) {
                const uint32_t G = min(4 * (q0 + s) + ig, ngroups - 1);
#pragma unroll
                for (int b = 0; b < BP; b++) xr[s][b] = xa.xq[(G * 16 + j) * BP + b];
            }
        }
        // ---- 2. block scales (one load per quad), then the quants
        uint2 sr[QPW];
        uint4 qa[QPW][4], qb8[Q4 ? 1 : QPW][Q4 ? 1 : 4];
        typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
#pragma unroll
        for (int s = 0; s < QPW; s++) {
            const uint32_t G = min(4 * (q0 + s) + ig, ngroups - 1);
            const u32x2_t sv = __builtin_nontemporal_load((const u32x2_t *)(ds + (cb + G) * 16 + j));
            sr[s] = make_uint2(sv.x, sv.y);
        }
#pragma unroll
        for (int s = 0; s < QPW; s++)
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const uint64_t c = cb + min(4 * (q0 + s) + u, ngroups - 1);
                if (Q4) {
                    qa[s][u] = load_stream(qs + c * 64 + lane);
                } else {
                    qa[s][u] = load_stream(qs + (c * 2) * 64 + lane);
                    qb8[Q4 ? 0 : s][Q4 ? 0 : u] = load_stream(qs + (c * 2 + 1) * 64 + lane);
                }
            }
        {   // (no branch here: a branch between the requests and their first use makes the compiler wait for all of them)
            const uint32_t inner = kv_inner ? kv_inner : 16u, hd = e.kv_hd ? e.kv_hd : 16u;
            const uint32_t c = (T * 16) % inner, hh = c / hd, d0 = c % hd;
            kv_idx = (((uint64_t)ig * e.kv_heads + hh) * e.kv_max_ctx + kvpos) * hd + d0 + j;
        }
        // ---- 3. stage this wave's activation pieces (the weights are still on their way)
        if constexpr (NORM) {
            if (wave == 0) {
                // mean = sum(s_t) / k, k * var = sum(M2_t + c_t * (s_t / c_t - mean)^2); with mean = 0 the
                // same expression is sum(x^2), which is what the RMS norm divides by.  Hardware
                // reciprocal and reciprocal square root (1 ulp): the result is rounded to f16.
                const float rk = __builtin_amdgcn_rcpf((float)k);
                const uint32_t tail = k & 15;
                const float rc_tail = tail ? __builtin_amdgcn_rcpf((float)tail) : 0.0625f;
#pragma unroll
                for (int b = 0; b < BP; b++) {
                    float sm = 0.f;
#pragma unroll
                    for (int u = 0; u < SREC; u++) sm += lane + 64 * u < nt ? rec0[b][u].x : 0.f;
                    const float mean = RMS ? 0.f : wave_sum(sm) * rk;
                    float q = 0.f;
#pragma unroll
                    for (int u = 0; u < SREC; u++) {
                        const uint32_t t = lane + 64 * u;
                        const bool last = tail && t == nt - 1;
                        const float c = last ? (float)tail : 16.f, rc = last ? rc_tail : 0.0625f;
                        const float d = rec0[b][u].x * rc - mean;
                        q += t < nt ? fmaf(c * d, d, rec0[b][u].y) : 0.f;
                    }
                    const float rsd = __builtin_amdgcn_rsqf(wave_sum(q) * rk + xa.eps);
                    if (lane == 0) rowstat[b] = make_float2(mean, rsd);
                }
            }
            lds_barrier();
            const uint32_t G = 4 * q0 + ig;
            const bool piece_live = G < ngroups && (G * 16 + j) * 8 < k;
            float sc[8];
            if (PRE) {
#pragma unroll
                for (int u = 0; u < 8; u++) sc[u] = 1.f;
            } else {
                const float t[8] = {scv[0].x, scv[0].y, scv[0].z, scv[0].w, scv[1].x, scv[1].y, scv[1].z, scv[1].w};
#pragma unroll
                for (int u = 0; u < 8; u++) sc[u] = t[u];
            }
#pragma unroll
            for (int b = 0; b < BP; b++) {
                const float2 ms = rowstat[b];
                const float v[8] = {hv[b][0].x, hv[b][0].y, hv[b][0].z, hv[b][0].w,
                                    hv[b][1].x, hv[b][1].y, hv[b][1].z, hv[b][1].w};
                float y[8];
#pragma unroll
                for (int u = 0; u < 8; u++) y[u] = (v[u] - ms.x) * (sc[u] * ms.y);  // scale * (x - mean) / sd (MT:124)
                if (!RMS) {
                    const float bi[8] = {biv[0].x, biv[0].y, biv[0].z, biv[0].w, biv[1].x, biv[1].y, biv[1].z, biv[1].w};
#pragma unroll
                    for (int u = 0; u < 8; u++) y[u] += bi[u];
                }
                union { uint4 u; half2_t h2[4]; } o;
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    o.h2[u].x = (_Float16)y[2 * u];
                    o.h2[u].y = (_Float16)y[2 * u + 1];
                }
                if (!(piece_live && (uint32_t)b < batch)) o.u = make_uint4(0, 0, 0, 0);
                float sx;
                xw[(ig * 16 + j) * BP + b] = quad_piece<Q4>(o.u, sx);
                sx += dpp_f32<DPP_QUAD_XOR1>(sx);
                sx += dpp_f32<DPP_QUAD_XOR2>(sx);  // the block = four neighbouring pieces
                if ((j & 3) == 0) sw[(ig * 4 + (j >> 2)) * BP + b] = (Q4 ? -8.f : -128.f) * sx;
            }
        } else {
#pragma unroll
            for (int s = 0; s < QPW; s++)
#pragma unroll
                for (int b = 0; b < BP; b++) {
                    float sx;
                    xw[((s * 4 + ig) * 16 + j) * BP + b] = quad_piece<Q4>(xr[s][b], sx);
                    sx += dpp_f32<DPP_QUAD_XOR1>(sx);
                    sx += dpp_f32<DPP_QUAD_XOR2>(sx);
                    if ((j & 3) == 0) sw[((s * 4 + ig) * 4 + (j >> 2)) * BP + b] = (Q4 ? -8.f : -128.f) * sx;
                }
        }
        // ---- 4. products
#pragma unroll
        for (int s = 0; s < QPW; s++) {
            union { uint2 u2; half2_t h[2]; } scu;
            scu.u2 = sr[s];
            const bool chunk_live = 4 * (q0 + s) + ig < ngroups;  // a chunk past the end was re-read: no weight
            float d[4] = {(float)scu.h[0].x, (float)scu.h[0].y, (float)scu.h[1].x, (float)scu.h[1].y};
#pragma unroll
            for (int jj = 0; jj < 4; jj++) d[jj] = chunk_live ? d[jj] : 0.f;
            // this lane group's own chunk: the offset term d * (-8 S) of its four blocks
#pragma unroll
            for (int jj = 0; jj < 4; jj++)
#pragma unroll
                for (int i = 0; i < NI; i++) acc[i] = fmaf(d[jj], sw[((s * 4 + ig) * 4 + jj) * BP + i], acc[i]);
            float dm[4];  // the nibbles entered as n * 2^-24
#pragma unroll
            for (int jj = 0; jj < 4; jj++) dm[jj] = d[jj] * 16777216.f;
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const uint32_t qw[8] = {qa[s][u].x, qa[s][u].y, qa[s][u].z, qa[s][u].w,
                                        Q4 ? 0u : qb8[Q4 ? 0 : s][Q4 ? 0 : u].x, Q4 ? 0u : qb8[Q4 ? 0 : s][Q4 ? 0 : u].y,
                                        Q4 ? 0u : qb8[Q4 ? 0 : s][Q4 ? 0 : u].z, Q4 ? 0u : qb8[Q4 ? 0 : s][Q4 ? 0 : u].w};
#pragma unroll
                for (int jj = 0; jj < 4; jj++) {
                    union { uint4 u4; half8_t h; } xv;
                    xv.u4 = xw[((s * 4 + u) * 16 + 4 * jj + ig) * BP + (j & (BP - 1))];
                    const half8_t wv = Q4 ? quad_operand<true>(qw[jj], 0u) : quad_operand<false>(qw[2 * jj], qw[2 * jj + 1]);
                    const float4_t part = __builtin_amdgcn_mfma_f32_16x16x32_f16(xv.h, wv, zero, 0, 0, 0);
                    if (ig == (uint32_t)u) {
#pragma unroll
                        for (int i = 0; i < NI; i++) acc[i] = fmaf(dm[jj], part[i], acc[i]);
                    }
                }
            }
        }
    }

    // ---- 5. the four lane groups, then the waves, meet; wave 0 finishes the tile
#pragma unroll
    for (int i = 0; i < NI; i++) {
        const float v = xor32_sum(xor16_sum(acc[i]));
        if (ig == 0) red[(wave * NI + i) * 16 + j] = v;
    }
    lds_barrier();
    if (wave != 0) return;
    const uint32_t b = ig;  // this lane's batch row
    float a = 0.f;
    if (b < (uint32_t)NI)
        for (uint32_t w = 0; w < nwaves; w++) a += red[(w * NI + b) * 16 + j];
    const bool live = b < (uint32_t)NI && b < batch && col < ep_n;
    if (kv_odd) {  // q|k|v of sizes that are not multiples of 16: the general walk
        if (live) epi_store<true>(e, b, col, a, true, res_pre, true, kvpos);
        return;
    }
    a += bias_pre;
    if (gated) {
        // weight rows (2m, 2m+1) = (gate_m, up_m) sit in neighbouring lanes
        const float up = lane_xor1(a);
        if (live && (lane & 1) == 0) {
            const uint64_t m = col >> 1;
            float v = fast_silu(a) * up;
            if (e.residual) v += e.residual[(uint64_t)b * n_eff + m];
            if (out_f32) out_f32[(uint64_t)b * n_eff + m] = v;
            if (out_xq) out_xq[xq_index(m, b, bp_out)] = __float2half_rn(v);
            if (out_lp) out_lp[(uint64_t)b * lp_ld + m] = f32_to_lp_bits(v, lp_bf16);
        }
        return;
    }
    if (kv_tile) {  // key or value columns: into the cache, nothing else
        if (live) kv_cache_store(T * 16 < 2 * kv_inner ? kv_k : kv_v, kv_dtype, kv_idx, a);
        return;
    }
    if (ep_act == COEUS_EPI_GELU) a = fast_gelu(a);
    const float v = a + res_pre;
    const uint64_t oidx_g = (uint64_t)b * n_eff + col;
    if (live) {
        if (out_f32) out_f32[(uint64_t)b * n_eff + col] = v;
        if (out_xq) out_xq[xq_index(col, b, bp_out)] = __float2half_rn(v);
        if (out_lp) out_lp[(uint64_t)b * lp_ld + col] = f32_to_lp_bits(v, lp_bf16);
        if (e.g_out) e.g_out[oidx_g] = v * gs_pre;  // the copy that the next norm's matmul stages
    }
    if (stats_out) {  // uniform; never combined with the gated epilogue
        const uint32_t left = (uint32_t)ep_n - T * 16;
        const float2 r = group16_stats(live ? v : 0.f, live, left < 16 ? left : 16u);
        if (j == 0 && b < (uint32_t)NI && b < batch) stats_out[(uint64_t)b * stats_tiles + T] = r;
    }
}

static const size_t kXLdsLimit = 48 * 1024;

// Waves per workgroup of gemv_quant_kernel: enough waves to cover the chip several times over, at
// least 2 chunks per wave.
static uint32_t gemv_quant_waves(const Weight &w) {
    const uint32_t ngroups = (uint32_t)(w.k_pad / 128), tiles = (uint32_t)(w.n_pad / 16);
    uint32_t waves = 4;
    while (waves < 16 && (uint64_t)tiles * waves < 4096 && ngroups >= waves * 4) waves *= 2;
    while (waves > 1 && waves > ngroups) waves /= 2;
    return waves;
}

bool gemv_can_fuse_norm(const Weight &w, uint64_t batch) {
    if (w.dtype < COEUS_W_Q8_0 || batch < 1 || batch > 16) return false;
    const uint32_t bp = pad_batch(batch);
    // (gemv_quad_kernel: one quad of 512 k per wave, at most 16 waves; 4 or 8 statistics records
    // per lane and row, 8 only for up to two rows)
    return bp <= 4 && (w.k & 7) == 0 && w.k <= 16u * 64u * 8u && w.k_pad * bp * 2 <= kXLdsLimit &&
           (bp < 4 || w.k <= 16u * 64u * 4u);
}

struct GemvLaunch {
    dim3 grid, block;
    size_t lds;
    hipStream_t st;
    const uint4 *qs;
    const uint2 *ds;
    XArgs xa;
    uint32_t ngroups, tiles, batch;
    EpiArgs e;
};

template <bool Q4, int BPV, int MODE, int CFG>
static void gemv_launch_one(const GemvLaunch &L) {
    hipLaunchKernelGGL((gemv_quant_kernel<Q4, BPV, MODE, CFG>), L.grid, L.block, L.lds, L.st, L.qs,
                       L.ds, L.xa, L.ngroups, L.tiles, L.batch, L.e);
}

template <bool Q4, int BPV, int MODE>
static bool gemv_launch_cfg(int cfg, const GemvLaunch &L) {
    switch (cfg) {
        case 1: gemv_launch_one<Q4, BPV, MODE, 1>(L); return true;
        case 1 | CFG_TPW2: if constexpr (MODE == X_LDS) { gemv_launch_one<Q4, BPV, MODE, 1 | CFG_TPW2>(L); return true; } return false;
        case 1 | CFG_TPW4: if constexpr (MODE == X_GLOBAL) { gemv_launch_one<Q4, BPV, MODE, 1 | CFG_TPW4>(L); return true; } return false;
        case 1 | CFG_PF6: gemv_launch_one<Q4, BPV, MODE, 1 | CFG_PF6>(L); return true;
        case 1 | CFG_PF2: gemv_launch_one<Q4, BPV, MODE, 1 | CFG_PF2>(L); return true;
        default: return false;
    }
}

template <bool Q4, int BPV>
static bool gemv_launch_mode(int xmode, int cfg, const GemvLaunch &L) {
    return xmode == X_GLOBAL ? gemv_launch_cfg<Q4, BPV, X_GLOBAL>(cfg, L) : gemv_launch_cfg<Q4, BPV, X_LDS>(cfg, L);
}

template <bool Q4, int BPV, int MODE, int QPWV, int SRECV>
static bool quad_launch_one(const GemvLaunch &L) {
    const void *kern = (const void *)gemv_quad_kernel<Q4, BPV, MODE, QPWV, SRECV>;
    if (L.lds > 48 * 1024) {
        static const hipError_t once = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (once != hipSuccess) return false;
    }
    hipLaunchKernelGGL((gemv_quad_kernel<Q4, BPV, MODE, QPWV, SRECV>), L.grid, L.block, L.lds, L.st, L.qs, L.ds, L.xa,
                       L.ngroups, L.tiles, L.batch, L.e);
    return true;
}

template <bool Q4, int BPV>
static bool quad_launch_bp(int xmode, uint32_t qpw, uint32_t srec, const GemvLaunch &L) {
    if (xmode == X_LDS) return qpw == 1 ? quad_launch_one<Q4, BPV, X_LDS, 1, 4>(L) : quad_launch_one<Q4, BPV, X_LDS, 2, 4>(L);
    if (qpw != 1) return false;
    if (xmode == X_LAYERNORM) {
        if (srec == 4) return quad_launch_one<Q4, BPV, X_LAYERNORM, 1, 4>(L);
        if constexpr (BPV <= 2) return quad_launch_one<Q4, BPV, X_LAYERNORM, 1, 8>(L);
        return false;
    }
    if (xmode == X_RMSPRE) {
        if (srec == 4) return quad_launch_one<Q4, BPV, X_RMSPRE, 1, 4>(L);
        if constexpr (BPV <= 2) return quad_launch_one<Q4, BPV, X_RMSPRE, 1, 8>(L);
        return false;
    }
    if (srec == 4) return quad_launch_one<Q4, BPV, X_RMSNORM, 1, 4>(L);
    if constexpr (BPV <= 2) return quad_launch_one<Q4, BPV, X_RMSNORM, 1, 8>(L);
    return false;
}

// Batches of up to 4: gemv_quad_kernel, one workgroup per tile of 16 rows.  A wave takes quads of
// four chunks; with a folded norm one quad per wave and as many waves as the reduction has quads;
// plain activations: one or two quads in flight per wave, several passes when 16 waves do not cover
// k that way.
template <bool Q4>
static int launch_gemv_quad(const Weight &w, const __half *xq, uint64_t batch, const EpiArgs &e, hipStream_t st,
                            const NormFuse *nf) {
    const uint32_t ngroups = (uint32_t)(w.k_pad / 128), tiles = (uint32_t)(w.n_pad / 16);
    const uint32_t bp = pad_batch(batch), nquads = (ngroups + 3) / 4;
    if (nf && (!gemv_can_fuse_norm(w, batch) || !nf->stats))
        return fail(COEUS_INVALID_INPUT, "norm fusion needs the activations to fit in LDS and the "
                                         "producer's statistics records");
    if (e.stats_out && e.act == COEUS_EPI_SILU_GATE)
        return fail(COEUS_INVALID_INPUT, "statistics records are not produced by the gated epilogue");
    XArgs xa{};
    xa.xq = (const uint4 *)xq;
    xa.k = (uint32_t)w.k;
    int xmode = X_LDS;
    uint32_t qpw = 1, waves = nquads, srec = 4;
    if (nf) {
        xmode = nf->kind == COEUS_NORM_RMSNORM ? X_RMSNORM : X_LAYERNORM;
        xa.h = nf->h; xa.nscale = nf->scale; xa.nbias = nf->bias; xa.stats = nf->stats; xa.eps = nf->eps;
        srec = w.k > 16u * 64u * 4u ? 8 : 4;
        if (nf->g) {
            if (xmode != X_RMSNORM) return fail(COEUS_INVALID_INPUT, "pre-scaled rows are for a root-mean-square norm");
            xmode = X_RMSPRE;
            xa.h = nf->g;
        }
    } else if (nquads > 16) {
        qpw = 2;
        const uint32_t passes = (nquads + 31) / 32;
        waves = (nquads + 2 * passes - 1) / (2 * passes);
    }
    // every wave keeps its activation pieces in LDS: at most 64 KiB of them per workgroup
    const size_t wbytes = (size_t)qpw * bp * 68 * 16;
    while (waves > 1 && waves * wbytes > 64 * 1024) waves = (waves + 1) / 2;
    GemvLaunch L;
    L.grid = dim3(tiles);
    L.block = dim3(waves * 64);
    L.lds = waves * wbytes + (size_t)waves * bp * 16 * 4 + bp * 8;
    L.st = st;
    L.qs = (const uint4 *)w.data;
    L.ds = (const uint2 *)w.scales;
    L.xa = xa;
    L.ngroups = ngroups; L.tiles = tiles; L.batch = (uint32_t)batch;
    L.e = e;
    bool ok;
    switch (bp) {
        case 1: ok = quad_launch_bp<Q4, 1>(xmode, qpw, srec, L); break;
        case 2: ok = quad_launch_bp<Q4, 2>(xmode, qpw, srec, L); break;
        default: ok = quad_launch_bp<Q4, 4>(xmode, qpw, srec, L); break;
    }
    if (!ok) return fail(COEUS_INVALID_INPUT, "decode matmul: no quad kernel for mode %d and %u quads per wave", xmode, qpw);
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

template <bool Q4>
static int launch_gemv_quant(const Weight &w, const __half *xq, uint64_t batch, const EpiArgs &e,
                             hipStream_t st, const NormFuse *nf) {
    if (pad_batch(batch) <= 4) return launch_gemv_quad<Q4>(w, xq, batch, e, st, nf);
    // batches of 5 to 16: gemv_quant_kernel on staged f16 activations (the norm is a launch of its own)
    if (nf) return fail(COEUS_INVALID_INPUT, "norm fusion is for batches of up to 4");
    const uint32_t ngroups = (uint32_t)(w.k_pad / 128), tiles = (uint32_t)(w.n_pad / 16);
    const uint32_t bp = pad_batch(batch), b = (uint32_t)batch;
    uint32_t waves = gemv_quant_waves(w);
    const size_t x_bytes = (size_t)w.k_pad * bp * 2;
    const bool xlds = x_bytes <= kXLdsLimit;
    if (e.stats_out && e.act == COEUS_EPI_SILU_GATE)
        return fail(COEUS_INVALID_INPUT, "statistics records are not produced by the gated epilogue");
    const int xmode = xlds ? X_LDS : X_GLOBAL;
    XArgs xa{};
    xa.xq = (const uint4 *)xq;
    xa.k = (uint32_t)w.k;
    const uint32_t pf = Q4 ? 4 : 2;
    const bool one_pass = ngroups <= pf * waves;
    int cfg = 1;
    if (!one_pass && ngroups <= pf * waves * 3 / 2) {
        cfg |= CFG_PF6;  // one pass of 6 chunks per wave instead of a full and a partial pass
    } else if (ngroups <= (pf / 2) * waves) {
        cfg |= CFG_PF2;  // half as many chunks per wave cover k: no requests past the end
    }
    // two tiles per workgroup where one pass covers the reduction and the tiles still fill the
    // chip: the activation block is staged half as often
    uint32_t tpw = 1;
    if (xmode == X_GLOBAL) {
        // activations from L2: several tiles per workgroup share every activation fragment; the
        // waves split k finer instead, so that the chip still holds thousands of them
        tpw = tiles >= 768 ? 4 : 1;
        if (tpw > 1) {
            cfg = 1 | CFG_TPW4;
            waves = tiles / tpw < 256 ? 16 : 8;
            while (waves > 1 && waves * 2 > ngroups) waves /= 2;
        }
    } else if (one_pass && waves >= 2 && tiles >= 1024 && cfg == 1) {
        cfg |= CFG_TPW2;
        tpw = 2;
    }
    const size_t red_bytes = (waves > 1 || tpw > 1) ? (size_t)tpw * waves * 4 * 64 * 4 : 0;
    GemvLaunch L;
    L.grid = dim3((unsigned)ceil_div(tiles, tpw));
    L.block = dim3(waves * 64);
    L.lds = (xmode != X_GLOBAL ? x_bytes : 0) + red_bytes;
    L.st = st;
    L.qs = (const uint4 *)w.data;
    L.ds = (const uint2 *)w.scales;
    L.xa = xa;
    L.ngroups = ngroups; L.tiles = tiles; L.batch = b;
    L.e = e;
    const bool ok = bp == 8 ? gemv_launch_mode<Q4, 8>(xmode, cfg, L) : gemv_launch_mode<Q4, 16>(xmode, cfg, L);
    if (!ok) return fail(COEUS_INVALID_INPUT, "decode matmul: no kernel variant %d for mode %d", cfg, xmode);
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

// ---------------------------------------------------------------- dense kernel (f32 / bf16)
// One wave per output row.  NORM = 0: x is the activation block [batch, k] in global memory.
// NORM = 1 (LayerNorm) / 2 (RMSNorm): x is the residual stream; the workgroup (16 waves = 16 rows)
// normalises it once into LDS, evaluated like norm_token_kernel (scale * (x - mean) / sd + bias),
// and its waves read the normalised rows from there: no separate norm launch.  Wave b computes
// the statistics of batch row b on its own (two passes over the row), while every wave already
// has its first weights on the way.
template <bool BF16, int BP, int NORM>
__global__ __launch_bounds__(1024) void gemv_dense_kernel(const void *__restrict__ wdata,
                                                          const float *__restrict__ x, uint64_t k,
                                                          uint32_t batch, EpiArgs e,
                                                          const float *__restrict__ nscale,
                                                          const float *__restrict__ nbias, float eps) {
    extern __shared__ float xn[];  // NORM: [BP][k] rows, [2][k] scale and bias, partial sums, statistics
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    const uint64_t j = (uint64_t)blockIdx.x * nwaves + wave;
    const uint64_t jc = j < e.n ? j : e.n - 1;  // waves past the end repeat the last row (no early
                                                // return: every wave takes part in the barriers)
    float acc[BP];
#pragma unroll
    for (int b = 0; b < BP; b++) acc[b] = 0.f;
    const bool vec = (k & 7) == 0;
    // The first two steps of the row (2 x 512 k) are requested before anything else, from clamped
    // addresses (a step past the end re-reads the last 8 weights and is not used).  Weights are read
    // once per step: non-temporal loads (250M bf16, batch 1: 0.358 -> 0.344 ms per step).
    auto wload = [&](uint64_t k0, uint4 &a, uint4 &b) {
        const uint64_t kc = k0 + 8 <= k ? k0 : k - 8;
        if (BF16) {
            a = load_stream((const uint4 *)((const uint16_t *)wdata + jc * k + kc));
        } else {
            a = load_stream((const uint4 *)((const float *)wdata + jc * k + kc));
            b = load_stream((const uint4 *)((const float *)wdata + jc * k + kc + 4));
        }
    };
    uint4 wa0 = make_uint4(0, 0, 0, 0), wb0 = wa0, wa1 = wa0, wb1 = wa0;
    if (vec) {
        wload((uint64_t)lane * 8, wa0, wb0);
        wload((uint64_t)lane * 8 + 512, wa1, wb1);
    }
    const float *xs = x;  // where the main loop reads activation row b: xs + b * k
    if (NORM) {
        // One trip to memory: the rows, the scale and the bias all go to LDS first; the two
        // statistics passes and the normalisation then work from there.
        float *gs = xn + (size_t)BP * k, *bs = gs + k;  // scale, bias
        float *red = bs + k;                            // [16 waves][BP] partial sums
        float *stat = red + 16 * BP;                    // [0][b] mean, [1][b] standard deviation
        float ps[BP];
#pragma unroll
        for (int b = 0; b < BP; b++) ps[b] = 0.f;
        for (uint64_t i = threadIdx.x; i < k; i += blockDim.x) {
            gs[i] = nscale[i];
            if (NORM == 1) bs[i] = nbias[i];
#pragma unroll
            for (int b = 0; b < BP; b++)
                if (b < (int)batch) {
                    const float v = x[(uint64_t)b * k + i];
                    xn[(uint64_t)b * k + i] = v;
                    ps[b] += v;
                }
        }
        // every wave's partial per row -> wave 0 finishes row b = lane
        auto finish = [&](float (&p)[BP]) -> float {
#pragma unroll
            for (int b = 0; b < BP; b++) {
                const float t = wave_sum(p[b]);
                if (lane == 0) red[wave * BP + b] = t;
            }
            __syncthreads();
            float tot = 0.f;
            if (wave == 0 && lane < BP)
                for (uint32_t w = 0; w < nwaves; w++) tot += red[w * BP + lane];
            return tot;
        };
        if (NORM == 1) {
            const float tot = finish(ps);
            if (wave == 0 && lane < BP) stat[lane] = tot / (float)k;
            __syncthreads();
        } else if (threadIdx.x < BP) {
            stat[threadIdx.x] = 0.f;  // a root-mean-square norm subtracts no mean
        }
#pragma unroll
        for (int b = 0; b < BP; b++) ps[b] = 0.f;
        if (NORM == 2) __syncthreads();  // the rows and the zero means are in LDS
        for (uint64_t i = threadIdx.x; i < k; i += blockDim.x)
#pragma unroll
            for (int b = 0; b < BP; b++)
                if (b < (int)batch) {
                    const float d = xn[(uint64_t)b * k + i] - stat[b];
                    ps[b] = fmaf(d, d, ps[b]);
                }
        {
            const float tot = finish(ps);
            if (wave == 0 && lane < BP) stat[16 + lane] = sqrtf(tot / (float)k + eps);
            __syncthreads();
        }
        for (uint64_t i = threadIdx.x; i < k; i += blockDim.x) {
            const float g = gs[i], bi = NORM == 1 ? bs[i] : 0.f;
#pragma unroll
            for (int b = 0; b < BP; b++)
                if (b < (int)batch)
                    xn[(uint64_t)b * k + i] = g * (xn[(uint64_t)b * k + i] - stat[b]) / stat[16 + b] + bi;
        }
        __syncthreads();
        xs = xn;
    }
    if (vec) {
        auto step = [&](uint64_t k0, const uint4 &ra, const uint4 &rb) {
            float wv[8];
            if (BF16) {
                const uint32_t r[4] = {ra.x, ra.y, ra.z, ra.w};
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    wv[2 * t] = __uint_as_float(r[t] << 16);
                    wv[2 * t + 1] = __uint_as_float(r[t] & 0xffff0000u);
                }
            } else {
                wv[0] = __uint_as_float(ra.x); wv[1] = __uint_as_float(ra.y);
                wv[2] = __uint_as_float(ra.z); wv[3] = __uint_as_float(ra.w);
                wv[4] = __uint_as_float(rb.x); wv[5] = __uint_as_float(rb.y);
                wv[6] = __uint_as_float(rb.z); wv[7] = __uint_as_float(rb.w);
            }
#pragma unroll
            for (int b = 0; b < BP; b++) {
                if (b < (int)batch) {
                    const float4 xa = *(const float4 *)(xs + (uint64_t)b * k + k0);
                    const float4 xb = *(const float4 *)(xs + (uint64_t)b * k + k0 + 4);
                    float s = acc[b];
                    s = fmaf(wv[0], xa.x, s); s = fmaf(wv[1], xa.y, s);
                    s = fmaf(wv[2], xa.z, s); s = fmaf(wv[3], xa.w, s);
                    s = fmaf(wv[4], xb.x, s); s = fmaf(wv[5], xb.y, s);
                    s = fmaf(wv[6], xb.z, s); s = fmaf(wv[7], xb.w, s);
                    acc[b] = s;
                }
            }
        };
        uint64_t k0 = (uint64_t)lane * 8;
        if (k0 < k) step(k0, wa0, wb0);
        if (k0 + 512 < k) step(k0 + 512, wa1, wb1);
        // longer rows: one step ahead
        if (k0 + 1024 < k) {
            k0 += 1024;
            wload(k0, wa0, wb0);
            for (; k0 < k; k0 += 512) {
                wload(k0 + 512, wa1, wb1);
                step(k0, wa0, wb0);
                wa0 = wa1; wb0 = wb1;
            }
        }
    } else {
        for (uint64_t kk = lane; kk < k; kk += 64) {
            const float wv = BF16 ? bf16_bits_to_f32(((const uint16_t *)wdata)[jc * k + kk])
                                  : ((const float *)wdata)[jc * k + kk];
#pragma unroll
            for (int b = 0; b < BP; b++)
                if (b < (int)batch) acc[b] = fmaf(wv, xs[(uint64_t)b * k + kk], acc[b]);
        }
    }
#pragma unroll
    for (int b = 0; b < BP; b++) acc[b] = wave_sum(acc[b]);
    if (e.act == COEUS_EPI_SILU_GATE) {
        // pair (gate_m, up_m) = rows (2m, 2m+1) live in neighbouring waves: go through LDS
        __shared__ float pair[16][16];
        if (lane == 0)
#pragma unroll
            for (int b = 0; b < BP; b++) pair[wave][b] = acc[b];
        __syncthreads();
        if ((wave & 1) == 0 && lane < batch && j + 1 < e.n)
            epi_store_gated(e, lane, j / 2, pair[wave][lane], pair[wave + 1][lane]);
        return;
    }
    if (lane == 0 && j < e.n)
#pragma unroll
        for (int b = 0; b < BP; b++)
            if (b < (int)batch) epi_store<true>(e, b, j, acc[b]);
}

static const size_t kDenseNormLdsLimit = 64 * 1024;
// rows + scale + bias + per-wave partial sums + statistics
static size_t gemv_dense_norm_lds(uint64_t k, uint32_t bp) { return ((size_t)(bp + 2) * k + 16 * bp + 32) * 4; }

// True when the dense decode matmul can take the normalisation into its staging: the normalised
// activation block [batch padded, k] f32 has to fit in LDS.
bool gemv_can_fuse_norm_dense(const Weight &w, uint64_t batch) {
    if (w.dtype >= COEUS_W_Q8_0 || batch < 1 || batch > 16) return false;
    return gemv_dense_norm_lds(w.k, pad_batch(batch)) <= kDenseNormLdsLimit;
}

template <bool BF16>
static int launch_gemv_dense(const Weight &w, const float *x, uint64_t batch, const EpiArgs &e,
                             hipStream_t st, const NormFuse *nf) {
    const uint32_t bp = pad_batch(batch), b = (uint32_t)batch;
    if (nf && !gemv_can_fuse_norm_dense(w, batch))
        return fail(COEUS_INVALID_INPUT, "norm fusion needs the normalised activations to fit in LDS");
    if (nf && (!nf->h || !nf->scale || (nf->kind == COEUS_NORM_LAYERNORM && !nf->bias)))
        return fail(COEUS_INVALID_INPUT, "null pointer argument");
    // plain: 4 rows per workgroup; folded norm: 16, so that the block is normalised once per 16 rows
    const uint32_t waves = nf ? 16 : 4;
    const dim3 grid((unsigned)ceil_div(w.n, waves)), block(waves * 64);
    const size_t lds = nf ? gemv_dense_norm_lds(w.k, bp) : 0;
    const int norm = !nf ? 0 : nf->kind == COEUS_NORM_RMSNORM ? 2 : 1;
    const float *xin = nf ? nf->h : x;
    const float *ns = nf ? nf->scale : nullptr, *nb = nf ? nf->bias : nullptr;
    const float eps = nf ? nf->eps : 0.f;
#define COEUS_GEMVD2(BPV, NV) \
    hipLaunchKernelGGL((gemv_dense_kernel<BF16, BPV, NV>), grid, block, lds, st, w.data, xin, w.k, b, e, ns, nb, eps)
#define COEUS_GEMVD(BPV) \
    do { if (norm == 0) COEUS_GEMVD2(BPV, 0); else if (norm == 1) COEUS_GEMVD2(BPV, 1); else COEUS_GEMVD2(BPV, 2); } while (0)
    switch (bp) {
        case 1: COEUS_GEMVD(1); break;
        case 2: COEUS_GEMVD(2); break;
        case 4: COEUS_GEMVD(4); break;
        case 8: COEUS_GEMVD(8); break;
        default: COEUS_GEMVD(16); break;
    }
#undef COEUS_GEMVD
#undef COEUS_GEMVD2
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
    if (e.g_out && (w.dtype < COEUS_W_Q8_0 || pad_batch(batch) > 4 || !e.g_scale || e.act == COEUS_EPI_SILU_GATE || e.kv_k))
        return fail(COEUS_INVALID_INPUT, "a pre-scaled copy of the output is written by the quantised decode matmul "
                                         "for batches of up to 4, without gate or cache append");
    switch (w.dtype) {
        case COEUS_W_F32: return launch_gemv_dense<false>(w, (const float *)x, batch, e, st, nf);
        case COEUS_W_BF16: return launch_gemv_dense<true>(w, (const float *)x, batch, e, st, nf);
        case COEUS_W_Q8_0: return launch_gemv_quant<false>(w, (const __half *)x, batch, e, st, nf);
        default: return launch_gemv_quant<true>(w, (const __half *)x, batch, e, st, nf);
    }
}

// ---------------------------------------------------------------- short prompts on quantised weights
// A prompt pass of up to 64 rows streams every weight once, like a decode step, so it should
// stream the Q4_0 / Q8_0 blocks and not their 3.5x larger f16 copies.  One workgroup takes 128
// weight rows (4 waves x 2 tiles of 16) over a share of at most GPW 128-wide k groups (blockIdx.y):
// all of its weights (2 x GPW chunks per wave) are requested first, the activation rows of the
// share (f16, from the previous kernel's 16-bit output) are staged in LDS once for all four
// waves, and after one barrier each wave unpacks its chunks to f16(q * d) (the same values as the
// f16 copies, so the results match the large-prompt path) and multiplies them with MT fragments
// of 16 activation rows (v_mfma_f32_16x16x32_f16; a fragment read from LDS feeds both tiles).
// No barrier and no request inside the multiply phase.  With more than one share the workgroups
// store bare partial products for gemm_split_reduce_kernel.
template <int GPW>
struct QsLayout {
    static constexpr int XLD = GPW * 128 + 8;  // LDS row stride in elements: + 8 keeps the 16-byte reads of 16 rows on distinct banks
};

template <bool Q4, int MT, int GPW>
__global__ __launch_bounds__(256) void gemm_qskinny_kernel(const uint16_t *__restrict__ a, uint64_t lda, uint32_t m,
                                                           const uint4 *__restrict__ qs,
                                                           const uint2 *__restrict__ ds, uint32_t tiles,
                                                           uint32_t ngroups, uint32_t splits, EpiArgs e) {
    constexpr int XLD = QsLayout<GPW>::XLD;
    extern __shared__ __attribute__((aligned(16))) uint16_t xs[];  // [MT * 16][XLD]
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t j = lane & 15, g = lane >> 4;
    const uint32_t split = blockIdx.y;
    const uint32_t gb = ngroups * split / splits, ge = ngroups * (split + 1) / splits;  // ge - gb <= GPW
    const uint32_t T0 = blockIdx.x * 8 + wave * 2;
    const uint64_t c0 = (uint64_t)min(T0, tiles - 1) * ngroups, c1 = (uint64_t)min(T0 + 1, tiles - 1) * ngroups;
    // Every load is unconditional (a load under a branch makes the compiler wait for all of them
    // before the first use): past the end of the share the last group is read again and multiplied
    // by a zero scale.
    ChunkRegs<Q4> rw[GPW][2];
#pragma unroll
    for (int d = 0; d < GPW; d++) {
        const uint32_t Gd = min(gb + d, ge - 1);
        load_chunk<Q4>(rw[d][0], qs, ds, c0 + Gd, lane);
        load_chunk<Q4>(rw[d][1], qs, ds, c1 + Gd, lane);
    }
    // activations: MT * 16 rows x GPW * 16 pieces of 16 bytes, 256 threads (rows past the end repeat
    // the last, groups past the share its last; m <= 64 rows: 32-bit offsets from the uniform base)
    constexpr int PPR = GPW * 16, NPT = MT * 16 * PPR / 256;  // pieces per row, pieces per thread
#pragma unroll
    for (int h = 0; h < NPT; h += 4) {
        uint4 v[4];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t p = tid + 256 * (h + q), row = p / PPR, pc = p % PPR;
            const uint32_t G = min(gb + pc / 16, ge - 1);
            v[q] = *(const uint4 *)(a + (min(row, m - 1) * (uint32_t)lda + G * 128 + (pc & 15) * 8));
        }
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t p = tid + 256 * (h + q), row = p / PPR, pc = p % PPR;
            *(uint4 *)(xs + row * XLD + pc * 8) = v[q];
        }
    }
    float4_t acc[2][MT];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int u = 0; u < MT; u++) acc[t][u] = float4_t{0.f, 0.f, 0.f, 0.f};
    lds_barrier();
    const uint16_t *xb = xs + j * XLD + g * 8;
#pragma unroll
    for (int d = 0; d < GPW; d++) {
        const _Float16 live = gb + d < ge ? (_Float16)1.0f : (_Float16)0.0f;
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            half8_t wv[2];
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const ChunkRegs<Q4> &r = rw[d][t];
                const uint32_t qw[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, Q4 ? 0u : r.q1.x, Q4 ? 0u : r.q1.y,
                                        Q4 ? 0u : r.q1.z, Q4 ? 0u : r.q1.w};
                union { uint2 u2; _Float16 h[4]; } sc;
                sc.u2 = r.s;
                const half8_t q = Q4 ? unpack_q4(qw[jj]) : unpack_q8(qw[2 * jj], qw[2 * jj + 1]);
                wv[t] = q * (sc.h[jj] * live);  // f16(q * d): one rounding, as in the dense f16 copy
            }
#pragma unroll
            for (int u = 0; u < MT; u++) {
                union { uint4 u4; half8_t h; } xv;
                xv.u4 = *(const uint4 *)(xb + u * 16 * XLD + d * 128 + jj * 32);
                acc[0][u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xv.h, wv[0], acc[0][u], 0, 0, 0);
                acc[1][u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xv.h, wv[1], acc[1][u], 0, 0, 0);
            }
        }
    }
    // lane (j, g) holds outputs (row 16 u + 4 g + i, column 16 T + j)
    if (splits > 1) {
        // Bare products into this share's plane (the usual case).  Through LDS, which is free now,
        // so that a row's 128 columns leave as 512 contiguous bytes instead of 16 floats per wave.
        constexpr uint32_t OLD = 132;  // floats per LDS row
        float *ts = (float *)xs;
        lds_barrier();  // (the last group's reads of xs are done)
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int u = 0; u < MT; u++)
#pragma unroll
                for (int i = 0; i < 4; i++)
                    ts[(16 * u + 4 * g + i) * OLD + wave * 32 + t * 16 + j] = acc[t][u][i];
        lds_barrier();
        float *plane = e.out_f32 + (uint64_t)split * m * e.n;
        const uint64_t colbase = (uint64_t)blockIdx.x * 128;
        const uint32_t c4 = (tid & 31) * 4;
        for (uint32_t row = tid >> 5; row < MT * 16 && row < m; row += 8) {
            const float4 v = *(const float4 *)(ts + row * OLD + c4);
            float *dst = plane + (uint64_t)row * e.n + colbase + c4;
            if ((e.n & 3) == 0 && colbase + c4 + 3 < e.n) {
                *(float4 *)dst = v;
            } else {
                const float vv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int q = 0; q < 4; q++)
                    if (colbase + c4 + q < e.n) dst[q] = vv[q];
            }
        }
        return;
    }
    const bool gated = e.act == COEUS_EPI_SILU_GATE;
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const uint32_t T = T0 + t;
        const uint64_t col = (uint64_t)T * 16 + j;
#pragma unroll
        for (int u = 0; u < MT; u++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t row = 16 * u + 4 * g + i;
                // gated: weight rows (2c, 2c+1) = (gate_c, up_c) sit in neighbouring lanes
                const float other = lane_xor1(acc[t][u][i]);
                if (T >= tiles || row >= m || col >= e.n) continue;
                if (!gated) epi_store<false>(e, row, col, acc[t][u][i]);
                else if ((lane & 1) == 0) epi_store_gated(e, row, col >> 1, acc[t][u][i], other);
            }
    }
}

// k groups per workgroup: 4, or 2 when that takes the launch to at least 512 workgroups (narrow matrices).
static uint32_t qskinny_gpw(const Weight &w) {
    const uint32_t ngroups = (uint32_t)(w.k_pad / 128), tiles = (uint32_t)(w.n_pad / 16);
    const uint32_t wgs = (tiles + 7) / 8;
    return wgs * ((ngroups + 3) / 4) >= 512 ? 4 : 2;
}
static uint32_t qskinny_splits(const Weight &w) {
    const uint32_t ngroups = (uint32_t)(w.k_pad / 128), gpw = qskinny_gpw(w);
    return (ngroups + gpw - 1) / gpw;
}

// Up to 64 rows: with 128 (8 fragments of 16 rows per wave) the kernel needs 348 registers and
// is slower than the 256x256 kernel on the f16 copies.  Matrices of at least 4 M weights: below
// (the 250M shape) the 256x256 kernel split along k is as fast or faster.
bool gemm_uses_qskinny(const Weight &w, uint64_t m) {
    return w.dtype >= COEUS_W_Q8_0 && m >= 1 && m <= 64 && w.k == w.k_pad && w.k >= 128 &&
           w.k * w.n >= 4000000ull;
}

uint64_t gemm_qskinny_scratch_bytes(const Weight &w, uint64_t m) {
    if (!gemm_uses_qskinny(w, m)) return 0;
    const uint32_t s = qskinny_splits(w);
    return s > 1 ? (uint64_t)s * m * w.n * 4 : 0;
}

// `plain` is the epilogue of a k-split launch (bare products into planes of `partials`); the caller
// runs the reduce kernel with the real epilogue afterwards.  Returns the number of shares used.
int launch_gemm_qskinny(const Weight &w, const uint16_t *a, uint64_t lda, uint64_t m, const EpiArgs &e,
                        float *partials, uint64_t partials_bytes, uint32_t *splits_out, hipStream_t st) {
    const uint32_t ngroups = (uint32_t)(w.k_pad / 128), tiles = (uint32_t)(w.n_pad / 16);
    const uint32_t splits = qskinny_splits(w);
    if (splits > 1 && (!partials || partials_bytes < (uint64_t)splits * m * w.n * 4))
        return fail(COEUS_INVALID_INPUT, "short-prompt matmul needs %llu bytes for its partial products",
                    (unsigned long long)((uint64_t)splits * m * w.n * 4));
    *splits_out = splits;
    EpiArgs ke = e;
    if (splits > 1) {
        Epilogue pe;
        pe.out_f32 = partials;
        ke = make_epi(pe, w.n);
    }
    const dim3 grid((tiles + 7) / 8, splits);
    const uint4 *qs = (const uint4 *)w.data;
    const uint2 *ds = (const uint2 *)w.scales;
    const bool q4 = w.dtype == COEUS_W_Q4_0;
#define COEUS_QS(Q4V, MTV, GPWV)                                                                        \
    do {                                                                                                \
        constexpr int lds_bytes = MTV * 16 * QsLayout<GPWV>::XLD * 2;                                    \
        static const bool once = [] {                                                                   \
            (void)hipFuncSetAttribute((const void *)gemm_qskinny_kernel<Q4V, MTV, GPWV>,                \
                                      hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);            \
            return true;                                                                                \
        }();                                                                                            \
        (void)once;                                                                                     \
        hipLaunchKernelGGL((gemm_qskinny_kernel<Q4V, MTV, GPWV>), grid, dim3(256), (size_t)lds_bytes, st, a, lda, \
                           (uint32_t)m, qs, ds, tiles, ngroups, splits, ke);                            \
    } while (0)
#define COEUS_QS3(MTV, GPWV) do { if (q4) COEUS_QS(true, MTV, GPWV); else COEUS_QS(false, MTV, GPWV); } while (0)
#define COEUS_QS2(MTV) do { if (gpw == 4) COEUS_QS3(MTV, 4); else COEUS_QS3(MTV, 2); } while (0)
    const uint32_t gpw = qskinny_gpw(w);
    if (m <= 32) COEUS_QS2(2);
    else COEUS_QS2(4);
#undef COEUS_QS3
#undef COEUS_QS2
#undef COEUS_QS
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

}  // namespace coeus
