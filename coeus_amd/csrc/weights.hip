// Device-resident linear weights: allocation, packing from the reference's [k_in, n_out] f32
// layout (b[l*n + j], MT:65) into the layouts the matmul kernels stream, block quantisation
// (GGML block_q8_0 / block_q4_0 value convention) and the counter-based synthetic generator.
#include "common.hpp"

// Everything in this file must reproduce the CPU arithmetic bit for bit (quantiser, generator):
// no a*b+c may be fused into an FMA.  The build compiles this file with -ffp-contract=off.

namespace coeus {

// ---------------------------------------------------------------- synthetic generator
__host__ __device__ static inline uint64_t splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

// z(seed, i): the sum of eight uniform 16-bit integers, centred and scaled to unit variance.
// Integer arithmetic and one f32 multiply: the same bits on any device.
__host__ __device__ static inline float synth_normal(uint64_t seed_mixed, uint64_t index) {
    const uint64_t a = splitmix64(seed_mixed ^ ((2 * index) * 0xD1342543DE82EF95ull + 1));
    const uint64_t b = splitmix64(seed_mixed ^ ((2 * index + 1) * 0xD1342543DE82EF95ull + 1));
    int s = 0;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        s += (int)((a >> (16 * j)) & 0xffff);
        s += (int)((b >> (16 * j)) & 0xffff);
    }
#if defined(__HIP_DEVICE_COMPILE__)
    return __fmul_rn((float)(s - 262140), 1.8688124e-05f);
#else
    return (float)(s - 262140) * 1.8688124e-05f;  // one multiply: nothing to contract
#endif
}

float synth_value_host(uint64_t seed, uint64_t index) {
    volatile float z = synth_normal(splitmix64(seed), index);  // keep the two multiplies apart
    return 0.02f * z;
}

// Element (l, j) of the matrix being packed (see WeightSource in common.hpp).
struct Src {
    const float *p;
    uint64_t seed_mixed, base, n_part, k;
    uint32_t interleave;
    __device__ float operator()(uint64_t l, uint64_t j) const {
        const uint64_t part = interleave ? (j & 1) : j / n_part;
        const uint64_t col = interleave ? (j >> 1) : j % n_part;
        const uint64_t idx = base + part * k * n_part + l * n_part + col;
        return p ? p[idx] : __fmul_rn(0.02f, synth_normal(seed_mixed, idx));
    }
};

__global__ void fill_seeded_kernel(float *dst, uint64_t n, uint64_t seed_mixed, uint64_t base,
                                   float mean) {
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float z = __fmul_rn(0.02f, synth_normal(seed_mixed, base + i));
    dst[i] = mean != 0.0f ? __fadd_rn(mean, z) : z;
}

int launch_fill_seeded(float *dst, uint64_t n, uint64_t seed, uint64_t base, float mean,
                       hipStream_t st) {
    if (n == 0) return COEUS_OK;
    hipLaunchKernelGGL(fill_seeded_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, st, dst,
                       n, splitmix64(seed), base, mean);
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

__device__ static inline uint16_t f32_to_bf16_rne(float x) {
    uint32_t u = __float_as_uint(x);
    if ((u & 0x7f800000u) == 0x7f800000u && (u & 0x007fffffu)) return (uint16_t)((u | 0x00400000u) >> 16);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

__global__ void f32_to_bf16_kernel(const float *src, uint16_t *dst, uint64_t n) {
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = f32_to_bf16_rne(src[i]);
}

int launch_f32_to_bf16(const float *src, uint16_t *dst, uint64_t n, hipStream_t st) {
    if (n == 0) return COEUS_OK;
    hipLaunchKernelGGL(f32_to_bf16_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, st, src,
                       dst, n);
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

// ---------------------------------------------------------------- dense packing ([k,n] -> [n][k])
template <bool BF16>
__global__ void pack_dense_kernel(Src src, void *dst, uint64_t k, uint64_t n) {
    // 32x32 tile transposed through LDS: reads run along j (contiguous in the source),
    // writes run along l (contiguous in the destination).
    __shared__ float tile[32][33];
    const uint64_t l0 = (uint64_t)blockIdx.x * 32, j0 = (uint64_t)blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 256 threads: 8 rows per pass
    for (int r = ty; r < 32; r += 8) {
        const uint64_t l = l0 + r, j = j0 + tx;
        tile[r][tx] = (l < k && j < n) ? src(l, j) : 0.0f;
    }
    __syncthreads();
    for (int r = ty; r < 32; r += 8) {
        const uint64_t j = j0 + r, l = l0 + tx;
        if (j < n && l < k) {
            const float v = tile[tx][r];
            if (BF16) ((uint16_t *)dst)[j * k + l] = f32_to_bf16_rne(v);
            else ((float *)dst)[j * k + l] = v;
        }
    }
}

template <bool BF16>
__global__ void unpack_dense_kernel(const void *src, float *dst, uint64_t k, uint64_t n) {
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= k * n) return;
    const uint64_t l = idx / n, j = idx % n;
    float v;
    if (BF16) v = __uint_as_float((uint32_t)((const uint16_t *)src)[j * k + l] << 16);
    else v = ((const float *)src)[j * k + l];
    dst[idx] = v;
}

// ---------------------------------------------------------------- quantised packing
// One thread quantises one 32-element block (row j, block b) and scatters it into the tile
// layout described in common.hpp.
__device__ static inline uint64_t scale_index(uint64_t T, uint64_t G, uint64_t ngroups, int r, int jj) {
    return ((T * ngroups + G) * 16 + r) * 4 + jj;
}

template <bool Q4>
__global__ void pack_quant_kernel(Src src, uint32_t *qs, __half *ds, uint64_t k, uint64_t n,
                                  uint64_t nblk_pad, uint64_t n_pad) {
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= nblk_pad * n_pad) return;
    // consecutive threads take consecutive rows j of one block b: source reads are contiguous
    const uint64_t b = idx / n_pad, j = idx % n_pad;
    const uint64_t ngroups = nblk_pad / 4;
    const uint64_t T = j / 16, G = b / 4;
    const int r = (int)(j % 16), jj = (int)(b % 4);
    const bool live = (j < n) && (b * 32 < k);
    float x[32];
#pragma unroll
    for (int t = 0; t < 32; t++) x[t] = live ? src(b * 32 + t, j) : 0.0f;
    int q[32];
    float d;
    if (Q4) {
        float amax = 0.0f, mx = 0.0f;
#pragma unroll
        for (int t = 0; t < 32; t++) {
            const float a = fabsf(x[t]);
            if (amax < a) { amax = a; mx = x[t]; }
        }
        d = __fdiv_rn(mx, -8.0f);
        const float id = d != 0.0f ? __fdiv_rn(1.0f, d) : 0.0f;
#pragma unroll
        for (int t = 0; t < 32; t++) {
            int v = (int)(signed char)(int)__fadd_rn(__fmul_rn(x[t], id), 8.5f);
            q[t] = v > 15 ? 15 : v;
        }
    } else {
        float amax = 0.0f;
#pragma unroll
        for (int t = 0; t < 32; t++) amax = fmaxf(amax, fabsf(x[t]));
        d = __fdiv_rn(amax, 127.0f);
        const float id = d != 0.0f ? __fdiv_rn(1.0f, d) : 0.0f;
#pragma unroll
        for (int t = 0; t < 32; t++) q[t] = (int)roundf(__fmul_rn(x[t], id));
    }
    // keep the f32 scale a value of its own: folding the multiply above into the conversion
    // (v_fma_mix with a +0 addend) would turn the -0.0 scale of an all-zero block into +0.0
    asm volatile("" : "+v"(d));
    ds[scale_index(T, G, ngroups, r, jj)] = __float2half_rn(d);
    const uint64_t chunk = T * ngroups + G;
    if (Q4) {
        // GGML stores element t (t<16) in the low nibble of byte t and element t+16 in the high
        // nibble; the dequantised VALUES are what the convention fixes.  On the device a dword
        // holds k = 8g..8g+7 at nibble positions [k0,k2,k4,k6,k1,k3,k5,k7].
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int *e = q + 8 * g;
            const uint32_t w = (uint32_t)e[0] | ((uint32_t)e[2] << 4) | ((uint32_t)e[4] << 8) |
                               ((uint32_t)e[6] << 12) | ((uint32_t)e[1] << 16) |
                               ((uint32_t)e[3] << 20) | ((uint32_t)e[5] << 24) |
                               ((uint32_t)e[7] << 28);
            qs[(chunk * 64 + (16 * g + r)) * 4 + jj] = w;
        }
    } else {
#pragma unroll
        for (int g = 0; g < 4; g++)
#pragma unroll
            for (int dd = 0; dd < 2; dd++) {
                const int *e = q + 8 * g + 4 * dd;
                const uint32_t w = ((uint32_t)e[0] & 0xff) | (((uint32_t)e[1] & 0xff) << 8) |
                                   (((uint32_t)e[2] & 0xff) << 16) | (((uint32_t)e[3] & 0xff) << 24);
                qs[((chunk * 2 + (jj >> 1)) * 64 + (16 * g + r)) * 4 + (jj & 1) * 2 + dd] = w;
            }
    }
}

template <bool Q4>
__global__ void unpack_quant_kernel(const uint32_t *qs, const __half *ds, float *dst, uint64_t k,
                                    uint64_t n, uint64_t nblk_pad) {
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t nblk = k / 32;
    if (idx >= nblk * n) return;
    const uint64_t b = idx / n, j = idx % n;
    const uint64_t ngroups = nblk_pad / 4;
    const uint64_t T = j / 16, G = b / 4, chunk = T * ngroups + G;
    const int r = (int)(j % 16), jj = (int)(b % 4);
    const float d = __half2float(ds[scale_index(T, G, ngroups, r, jj)]);
#pragma unroll
    for (int g = 0; g < 4; g++) {
        if (Q4) {
            const uint32_t w = qs[(chunk * 64 + (16 * g + r)) * 4 + jj];
            const int pos[8] = {0, 4, 1, 5, 2, 6, 3, 7};  // nibble position of k-offset e
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int qv = (int)((w >> (4 * pos[e])) & 0xf) - 8;
                dst[(b * 32 + 8 * g + e) * n + j] = (float)qv * d;
            }
        } else {
#pragma unroll
            for (int dd = 0; dd < 2; dd++) {
                const uint32_t w = qs[((chunk * 2 + (jj >> 1)) * 64 + (16 * g + r)) * 4 + (jj & 1) * 2 + dd];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int qv = (int)(signed char)((w >> (8 * e)) & 0xff);
                    dst[(b * 32 + 8 * g + 4 * dd + e) * n + j] = (float)qv * d;
                }
            }
        }
    }
}

// Dense f16 [n][k] copy of a quantised weight for the prefill matmul: value = f16(q * d).
template <bool Q4>
__global__ void dequant_f16_kernel(const uint32_t *qs, const __half *ds, __half *dst, uint64_t k,
                                   uint64_t n, uint64_t nblk_pad, uint64_t ld) {
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t nblk = k / 32;
    if (idx >= nblk * n) return;
    // consecutive threads take consecutive blocks of one row: 64 B contiguous stores each
    const uint64_t j = idx / nblk, b = idx % nblk;
    const uint64_t ngroups = nblk_pad / 4;
    const uint64_t T = j / 16, G = b / 4, chunk = T * ngroups + G;
    const int r = (int)(j % 16), jj = (int)(b % 4);
    const float d = __half2float(ds[scale_index(T, G, ngroups, r, jj)]);
    __half *o = dst + j * ld + b * 32;
#pragma unroll
    for (int g = 0; g < 4; g++) {
        if (Q4) {
            const uint32_t w = qs[(chunk * 64 + (16 * g + r)) * 4 + jj];
            const int pos[8] = {0, 4, 1, 5, 2, 6, 3, 7};
#pragma unroll
            for (int e = 0; e < 8; e++)
                o[8 * g + e] = __float2half_rn((float)((int)((w >> (4 * pos[e])) & 0xf) - 8) * d);
        } else {
#pragma unroll
            for (int dd = 0; dd < 2; dd++) {
                const uint32_t w = qs[((chunk * 2 + (jj >> 1)) * 64 + (16 * g + r)) * 4 + (jj & 1) * 2 + dd];
#pragma unroll
                for (int e = 0; e < 4; e++)
                    o[8 * g + 4 * dd + e] = __float2half_rn((float)(int)(signed char)((w >> (8 * e)) & 0xff) * d);
            }
        }
    }
}

int launch_dequant_to_f16(const Weight &w, __half *dst_nk, uint64_t ld, hipStream_t st) {
    dim3 grid((unsigned)ceil_div(w.k / 32 * w.n, 256));
    if (w.dtype == COEUS_W_Q4_0)
        hipLaunchKernelGGL(dequant_f16_kernel<true>, grid, dim3(256), 0, st, (const uint32_t *)w.data,
                           w.scales, dst_nk, w.k, w.n, w.k_pad / 32, ld);
    else if (w.dtype == COEUS_W_Q8_0)
        hipLaunchKernelGGL(dequant_f16_kernel<false>, grid, dim3(256), 0, st, (const uint32_t *)w.data,
                           w.scales, dst_nk, w.k, w.n, w.k_pad / 32, ld);
    else
        return fail(COEUS_INVALID_INPUT, "dequant_to_f16 needs a quantised weight");
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

template <bool BF16>
__global__ void f32_to_16_kernel(const float *src, uint16_t *dst, uint64_t rows, uint64_t k, uint64_t ld) {
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * k) return;
    const uint64_t r = i / k, c = i % k;
    const float v = src[i];
    if (BF16) dst[r * ld + c] = f32_to_bf16_rne(v);
    else ((__half *)dst)[r * ld + c] = __float2half_rn(v);
}

int launch_f32_to_16(const float *src, void *dst, uint64_t rows, uint64_t k, uint64_t ld, bool bf16,
                     hipStream_t st) {
    if (rows * k == 0) return COEUS_OK;
    const dim3 grid((unsigned)ceil_div(rows * k, 256));
    if (bf16) hipLaunchKernelGGL(f32_to_16_kernel<true>, grid, dim3(256), 0, st, src, (uint16_t *)dst, rows, k, ld);
    else hipLaunchKernelGGL(f32_to_16_kernel<false>, grid, dim3(256), 0, st, src, (uint16_t *)dst, rows, k, ld);
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

// ---------------------------------------------------------------- host side
int weight_alloc(Weight &w, uint32_t dtype, uint64_t k, uint64_t n) {
    if (dtype > COEUS_W_Q4_0) return fail(COEUS_INVALID_INPUT, "unknown weight dtype %u", dtype);
    if (k == 0 || n == 0) return fail(COEUS_INVALID_INPUT, "empty weight %llu x %llu",
                                      (unsigned long long)k, (unsigned long long)n);
    w = Weight{};
    w.dtype = dtype;
    w.k = k;
    w.n = n;
    if (dtype == COEUS_W_F32 || dtype == COEUS_W_BF16) {
        w.k_pad = k;
        w.n_pad = n;
        w.bytes = k * n * (dtype == COEUS_W_F32 ? 4 : 2);
        COEUS_HIP(hipMalloc(&w.data, w.bytes));
        return COEUS_OK;
    }
    if (k % 32 != 0)
        return fail(COEUS_INVALID_INPUT,
                    "quantised weights need an input dimension divisible by 32, got %llu",
                    (unsigned long long)k);
    w.k_pad = round_up(k, 128);
    w.n_pad = round_up(n, 16);
    const uint64_t elems = w.k_pad * w.n_pad;
    const uint64_t qbytes = dtype == COEUS_W_Q4_0 ? elems / 2 : elems;
    const uint64_t sbytes = elems / 32 * 2;
    w.bytes = qbytes + sbytes;
    COEUS_HIP(hipMalloc(&w.data, qbytes));
    COEUS_HIP(hipMalloc((void **)&w.scales, sbytes));
    return COEUS_OK;
}

void weight_free(Weight &w) {
    if (w.data) (void)hipFree(w.data);
    if (w.scales) (void)hipFree(w.scales);
    if (w.xq_scratch) (void)hipFree(w.xq_scratch);
    if (w.expanded) (void)hipFree(w.expanded);
    w = Weight{};
}

int weight_expand(const Weight &w, uint64_t *budget, hipStream_t st) {
    if (w.dtype < COEUS_W_Q8_0 || w.expanded || !budget) return COEUS_OK;
    const uint64_t ld = gemm_ld(w.k), bytes = w.n * ld * 2;
    if (*budget < bytes) return COEUS_OK;
    void *p = nullptr;
    if (hipMalloc(&p, bytes) != hipSuccess) {  // no room: the matmul expands into its shared buffer
        (void)hipGetLastError();
        return COEUS_OK;
    }
    w.expanded = (__half *)p;
    *budget -= bytes;
    return launch_dequant_to_f16(w, w.expanded, ld, st);
}

int weight_pack(Weight &w, const WeightSource &ws, hipStream_t st) {
    Src src{ws.params, splitmix64(ws.seed), ws.base, ws.n_part ? ws.n_part : w.n, w.k, ws.interleave};
    if (w.dtype == COEUS_W_F32 || w.dtype == COEUS_W_BF16) {
        dim3 grid((unsigned)ceil_div(w.k, 32), (unsigned)ceil_div(w.n, 32));
        if (w.dtype == COEUS_W_BF16)
            hipLaunchKernelGGL(pack_dense_kernel<true>, grid, dim3(256), 0, st, src, w.data, w.k, w.n);
        else
            hipLaunchKernelGGL(pack_dense_kernel<false>, grid, dim3(256), 0, st, src, w.data, w.k, w.n);
    } else {
        const uint64_t nblk_pad = w.k_pad / 32, total = nblk_pad * w.n_pad;
        dim3 grid((unsigned)ceil_div(total, 64));
        if (w.dtype == COEUS_W_Q4_0)
            hipLaunchKernelGGL(pack_quant_kernel<true>, grid, dim3(64), 0, st, src,
                               (uint32_t *)w.data, w.scales, w.k, w.n, nblk_pad, w.n_pad);
        else
            hipLaunchKernelGGL(pack_quant_kernel<false>, grid, dim3(64), 0, st, src,
                               (uint32_t *)w.data, w.scales, w.k, w.n, nblk_pad, w.n_pad);
    }
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

int weight_unpack_to_device(const Weight &w, float *dst_kn, hipStream_t st) {
    if (w.dtype == COEUS_W_F32 || w.dtype == COEUS_W_BF16) {
        dim3 grid((unsigned)ceil_div(w.k * w.n, 256));
        if (w.dtype == COEUS_W_BF16)
            hipLaunchKernelGGL(unpack_dense_kernel<true>, grid, dim3(256), 0, st, w.data, dst_kn, w.k, w.n);
        else
            hipLaunchKernelGGL(unpack_dense_kernel<false>, grid, dim3(256), 0, st, w.data, dst_kn, w.k, w.n);
    } else {
        dim3 grid((unsigned)ceil_div(w.k / 32 * w.n, 64));
        if (w.dtype == COEUS_W_Q4_0)
            hipLaunchKernelGGL(unpack_quant_kernel<true>, grid, dim3(64), 0, st,
                               (const uint32_t *)w.data, w.scales, dst_kn, w.k, w.n, w.k_pad / 32);
        else
            hipLaunchKernelGGL(unpack_quant_kernel<false>, grid, dim3(64), 0, st,
                               (const uint32_t *)w.data, w.scales, dst_kn, w.k, w.n, w.k_pad / 32);
    }
    COEUS_HIP(hipGetLastError());
    return COEUS_OK;
}

}  // namespace coeus
