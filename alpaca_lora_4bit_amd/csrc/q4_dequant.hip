// Dense dequantization  out fp16 [K, N] = W   (HBM-bound: reads K*N/2 B, writes 2*K*N B).
//
// One thread owns one packed word-row (8 rows of W) x 8 adjacent columns: it reads 32 B of
// qweight with two 128-bit loads and writes eight 16-byte row segments, so a wavefront
// writes 1 KiB contiguous per row.  Scale / zero are re-fetched only when the row's group
// changes, which is never inside a word-row without act-order and up to 8 times with it.
//
// Values follow src/alpaca_lora_4bit/quant_cuda/quant_cuda_kernel.cu:1138-1152 bit for bit.
#include "q4_common.hpp"

namespace q4 {

__global__ __launch_bounds__(256) void dequant_kernel(
    const uint32_t* __restrict__ qweight, const uint32_t* __restrict__ qzeros,
    const half_t* __restrict__ scales, const int32_t* __restrict__ g_idx, int groupsize,
    half_t* __restrict__ out, int K, int N) {
    const int ncol8 = N >> 3;
    const long tid = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long total = (long)(K >> 3) * ncol8;
    if (tid >= total) return;
    const int kw = (int)(tid / ncol8);
    const int nb = (int)(tid - (long)kw * ncol8);
    const int n0 = nb << 3;

    const uint4_t* wp = reinterpret_cast<const uint4_t*>(qweight + (size_t)kw * N + n0);
    const uint4_t wa = wp[0], wb = wp[1];
    const uint32_t w[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};

    int gprev = -1;
    half2_t s2[4], zero2[4];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int k = (kw << 3) + e;
        const int g = g_idx ? g_idx[k] : k / groupsize;
        if (g != gprev) {
            gprev = g;
            const uint4_t sv = *reinterpret_cast<const uint4_t*>(scales + (size_t)g * N + n0);
            const uint32_t zw = qzeros[(size_t)g * ncol8 + nb];
            const uint32_t sraw[4] = {sv.x, sv.y, sv.z, sv.w};
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                s2[p] = as_half2(sraw[p]);
                zero2[p] = zero_term(s2[p], (zw >> (8 * p)) & 0xFu, (zw >> (8 * p + 4)) & 0xFu);
            }
        }
        uint32_t o[4];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const uint32_t codes = ((w[2 * p] >> (4 * e)) & 0xFu) | (((w[2 * p + 1] >> (4 * e)) & 0xFu) << 16);
            o[p] = as_u32(dequant_pair(codes_to_half2(codes), s2[p], zero2[p]));
        }
        uint4_t ov = {o[0], o[1], o[2], o[3]};
        __builtin_nontemporal_store(ov, reinterpret_cast<uint4_t*>(out + (size_t)k * N + n0));   // written once, not re-read here
    }
}

// fp32 flavour: scales fp32 [G, N], out fp32 [K, N]  (the float instantiation of the reference's template,
// src/alpaca_lora_4bit/quant_cuda/quant_cuda_kernel.cu:1126-1152, which _matmul4bit_v2_recons reaches when a model's
// scales were converted to float, matmul_utils_4bit.py:121-122).  zero = rn32(s * (z + 1)) and
// W = fma(s, q, -zero): one rounding for the product and the difference together, which is what the reference's build
// (nvcc defaults, setup.py passes no flags, so a * b - c contracts) computes; the separately rounded form differs from
// it by at most one unit in the last place.  Same thread mapping as dequant_kernel; HBM-bound on the 4*K*N B it writes.
__global__ __launch_bounds__(256) void dequant_f32_kernel(
    const uint32_t* __restrict__ qweight, const uint32_t* __restrict__ qzeros,
    const float* __restrict__ scales, const int32_t* __restrict__ g_idx, int groupsize,
    float* __restrict__ out, int K, int N) {
    const int ncol8 = N >> 3;
    const long tid = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long total = (long)(K >> 3) * ncol8;
    if (tid >= total) return;
    const int kw = (int)(tid / ncol8);
    const int nb = (int)(tid - (long)kw * ncol8);
    const int n0 = nb << 3;

    const uint4_t* wp = reinterpret_cast<const uint4_t*>(qweight + (size_t)kw * N + n0);
    const uint4_t wa = wp[0], wb = wp[1];
    const uint32_t w[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};

    int gprev = -1;
    float s[8], zero[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int k = (kw << 3) + e;
        const int g = g_idx ? g_idx[k] : k / groupsize;
        if (g != gprev) {
            gprev = g;
            const float4_t sa = *reinterpret_cast<const float4_t*>(scales + (size_t)g * N + n0);
            const float4_t sb = *reinterpret_cast<const float4_t*>(scales + (size_t)g * N + n0 + 4);
            const uint32_t zw = qzeros[(size_t)g * ncol8 + nb];
            s[0] = sa.x; s[1] = sa.y; s[2] = sa.z; s[3] = sa.w;
            s[4] = sb.x; s[5] = sb.y; s[6] = sb.z; s[7] = sb.w;
#pragma unroll
            for (int c = 0; c < 8; ++c) zero[c] = s[c] * (float)(((zw >> (4 * c)) & 0xFu) + 1u);
        }
        float o[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) o[c] = __builtin_fmaf(s[c], (float)((w[c] >> (4 * e)) & 0xFu), -zero[c]);
        float* dst = out + (size_t)k * N + n0;
        __builtin_nontemporal_store(float4_t{o[0], o[1], o[2], o[3]}, reinterpret_cast<float4_t*>(dst));
        __builtin_nontemporal_store(float4_t{o[4], o[5], o[6], o[7]}, reinterpret_cast<float4_t*>(dst + 4));
    }
}

// Row permutation of the packed weights: out row p holds the codes of input row perm[p].
// Used once per act-order layer to sort the rows by quantization group, after which the layer
// runs through the sequential-group kernels with x gathered through the same permutation.
// One thread per output word: eight nibbles gathered from eight source words (coalesced along N).
__global__ __launch_bounds__(256) void permute_rows_kernel(const uint32_t* __restrict__ qweight,
                                                           const int32_t* __restrict__ perm,
                                                           uint32_t* __restrict__ out, int K, int N) {
    const long tid = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long total = (long)(K >> 3) * N;
    if (tid >= total) return;
    const int kw = (int)(tid / N);
    const int n = (int)(tid - (long)kw * N);
    uint32_t word = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int k = perm[(kw << 3) + e];
        const uint32_t src = qweight[(size_t)(k >> 3) * N + n];
        word |= ((src >> ((k & 7) * 4)) & 0xFu) << (4 * e);
    }
    out[tid] = word;
}

// Column gather of an activation matrix: out[m, p] = in[m, idx[p]] (fp16, row-major [M, K]).  The companion of
// permute_rows_kernel at run time: x is gathered through the row sort before a product with the sorted weights, and
// grad_input is gathered back through the inverse permutation after it.  A workgroup stages `rows` whole rows in LDS
// with coalesced 16-byte loads and gathers from there (two-byte gathers from global memory cost one cache-line lookup
// per element), eight outputs per thread and row, written as 16-byte pieces.
__global__ __launch_bounds__(256) void permute_cols_kernel(const half_t* __restrict__ in, const int32_t* __restrict__ idx,
                                                           half_t* __restrict__ out, int M, int K, int rows) {
    extern __shared__ __attribute__((aligned(16))) half_t srow[];      // [rows][K]
    const int m0 = blockIdx.x * rows;
    const int nr = min(rows, M - m0);
    const int k8 = K >> 3;
    for (int i = threadIdx.x; i < nr * k8; i += 256)
        reinterpret_cast<uint4_t*>(srow)[i] = reinterpret_cast<const uint4_t*>(in + (size_t)m0 * K)[i];
    __syncthreads();
    for (int g = threadIdx.x; g < k8; g += 256) {
        const uint4_t i0 = *reinterpret_cast<const uint4_t*>(idx + 8 * g);
        const uint4_t i1 = *reinterpret_cast<const uint4_t*>(idx + 8 * g + 4);
        const uint32_t src[8] = {i0.x, i0.y, i0.z, i0.w, i1.x, i1.y, i1.z, i1.w};
        for (int r = 0; r < nr; ++r) {
            const unsigned short* row = reinterpret_cast<const unsigned short*>(srow) + r * K;
            uint32_t o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e)
                o[e] = (uint32_t)row[min(src[2 * e], (uint32_t)(K - 1))] | ((uint32_t)row[min(src[2 * e + 1], (uint32_t)(K - 1))] << 16);
            *reinterpret_cast<uint4_t*>(out + (size_t)(m0 + r) * K + 8 * g) = uint4_t{o[0], o[1], o[2], o[3]};
        }
    }
}

// v1 layout: one fp16 scale and one fp16 zero per column, W = rn16(rn16(s*q) - zero)
// (src/alpaca_lora_4bit/quant_cuda/quant_cuda_kernel.cu:1076-1097).  Same thread mapping as dequant_kernel.
__global__ __launch_bounds__(256) void dequant_v1_kernel(const uint32_t* __restrict__ qweight,
                                                         const half_t* __restrict__ scales,
                                                         const half_t* __restrict__ zeros,
                                                         half_t* __restrict__ out, int K, int N) {
    const int ncol8 = N >> 3;
    const long tid = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (tid >= (long)(K >> 3) * ncol8) return;
    const int kw = (int)(tid / ncol8);
    const int n0 = (int)(tid - (long)kw * ncol8) << 3;
    const uint4_t* wp = reinterpret_cast<const uint4_t*>(qweight + (size_t)kw * N + n0);
    const uint4_t wa = wp[0], wb = wp[1];
    const uint32_t w[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
    const uint4_t sv = *reinterpret_cast<const uint4_t*>(scales + n0);
    const uint4_t zv = *reinterpret_cast<const uint4_t*>(zeros + n0);
    const uint32_t sraw[4] = {sv.x, sv.y, sv.z, sv.w}, zraw[4] = {zv.x, zv.y, zv.z, zv.w};
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        uint32_t o[4];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const uint32_t codes = ((w[2 * p] >> (4 * e)) & 0xFu) | (((w[2 * p + 1] >> (4 * e)) & 0xFu) << 16);
            o[p] = as_u32(dequant_pair(codes_to_half2(codes), as_half2(sraw[p]), as_half2(zraw[p])));
        }
        *reinterpret_cast<uint4_t*>(out + (size_t)((kw << 3) + e) * N + n0) = uint4_t{o[0], o[1], o[2], o[3]};
    }
}

// 2-bit v2 layout: sixteen codes per word along K, sixteen zero codes per word along N, zero point = code + 1,
// W = rn16(rn16(s*q) - rn16(s*(z+1)))  (quant_cuda_kernel.cu:1185-1211).  One thread = one packed word-row
// (16 rows) x 8 columns.
__global__ __launch_bounds__(256) void dequant2_kernel(const uint32_t* __restrict__ qweight,
                                                       const uint32_t* __restrict__ qzeros,
                                                       const half_t* __restrict__ scales,
                                                       const int32_t* __restrict__ g_idx, int groupsize,
                                                       half_t* __restrict__ out, int K, int N) {
    const int ncol8 = N >> 3;
    const long tid = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (tid >= (long)(K >> 4) * ncol8) return;
    const int kw = (int)(tid / ncol8);
    const int nb = (int)(tid - (long)kw * ncol8);
    const int n0 = nb << 3;
    const uint4_t* wp = reinterpret_cast<const uint4_t*>(qweight + (size_t)kw * N + n0);
    const uint4_t wa = wp[0], wb = wp[1];
    const uint32_t w[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
    int gprev = -1;
    half2_t s2[4], zero2[4];
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        const int k = (kw << 4) + e;
        const int g = g_idx ? g_idx[k] : k / groupsize;
        if (g != gprev) {
            gprev = g;
            const uint4_t sv = *reinterpret_cast<const uint4_t*>(scales + (size_t)g * N + n0);
            // 8 adjacent columns are half of one packed zero word (16 codes of 2 bits)
            const uint32_t zw = qzeros[(size_t)g * (N >> 4) + (n0 >> 4)] >> ((n0 & 8) * 2);
            const uint32_t sraw[4] = {sv.x, sv.y, sv.z, sv.w};
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                s2[p] = as_half2(sraw[p]);
                zero2[p] = zero_term(s2[p], (zw >> (4 * p)) & 0x3u, (zw >> (4 * p + 2)) & 0x3u);
            }
        }
        uint32_t o[4];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const uint32_t codes = ((w[2 * p] >> (2 * e)) & 0x3u) | (((w[2 * p + 1] >> (2 * e)) & 0x3u) << 16);
            o[p] = as_u32(dequant_pair(codes_to_half2(codes), s2[p], zero2[p]));
        }
        *reinterpret_cast<uint4_t*>(out + (size_t)k * N + n0) = uint4_t{o[0], o[1], o[2], o[3]};
    }
}

}  // namespace q4

extern "C" int q4_launch_dequant_f32(const int32_t* qweight, const int32_t* qzeros, const float* scales,
                                     const int32_t* g_idx, int groupsize, float* out, int K, int N,
                                     hipStream_t stream) {
    const long total = (long)(K / 8) * (N / 8);
    hipLaunchKernelGGL(q4::dequant_f32_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                       reinterpret_cast<const uint32_t*>(qweight), reinterpret_cast<const uint32_t*>(qzeros),
                       scales, g_idx, groupsize, out, K, N);
    return hipGetLastError() == hipSuccess ? 0 : -4;
}

extern "C" int q4_launch_dequant_v1(const int32_t* qweight, const void* scales, const void* zeros, void* out,
                                    int K, int N, hipStream_t stream) {
    const long total = (long)(K / 8) * (N / 8);
    hipLaunchKernelGGL(q4::dequant_v1_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                       reinterpret_cast<const uint32_t*>(qweight), reinterpret_cast<const q4::half_t*>(scales),
                       reinterpret_cast<const q4::half_t*>(zeros), reinterpret_cast<q4::half_t*>(out), K, N);
    return hipGetLastError() == hipSuccess ? 0 : -4;
}

extern "C" int q4_launch_dequant2(const int32_t* qweight, const int32_t* qzeros, const void* scales,
                                  const int32_t* g_idx, int groupsize, void* out, int K, int N, hipStream_t stream) {
    const long total = (long)(K / 16) * (N / 8);
    hipLaunchKernelGGL(q4::dequant2_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                       reinterpret_cast<const uint32_t*>(qweight), reinterpret_cast<const uint32_t*>(qzeros),
                       reinterpret_cast<const q4::half_t*>(scales), g_idx, groupsize,
                       reinterpret_cast<q4::half_t*>(out), K, N);
    return hipGetLastError() == hipSuccess ? 0 : -4;
}

extern "C" int q4_launch_permute_rows(const int32_t* qweight, const int32_t* perm, int32_t* out, int K, int N,
                                      hipStream_t stream) {
    const long total = (long)(K / 8) * N;
    hipLaunchKernelGGL(q4::permute_rows_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                       reinterpret_cast<const uint32_t*>(qweight), perm, reinterpret_cast<uint32_t*>(out), K, N);
    return hipGetLastError() == hipSuccess ? 0 : -4;
}

// Rows per workgroup: as many as 64 KB of LDS hold, fewer when that would leave CUs without a workgroup.
extern "C" int q4_launch_permute_cols(const void* in, const int32_t* idx, void* out, int M, int K, hipStream_t stream) {
    const int fit = (64 * 1024) / (K * 2);
    if (fit < 1) return -2;
    int rows = fit > 16 ? 16 : fit;
    while (rows > 1 && (M + rows - 1) / rows < 512) --rows;
    hipLaunchKernelGGL(q4::permute_cols_kernel, dim3((unsigned)((M + rows - 1) / rows)), dim3(256), (size_t)rows * K * 2, stream,
                       reinterpret_cast<const q4::half_t*>(in), idx, reinterpret_cast<q4::half_t*>(out), M, K, rows);
    return hipGetLastError() == hipSuccess ? 0 : -4;
}

extern "C" int q4_launch_dequant(const int32_t* qweight, const int32_t* qzeros, const void* scales,
                                 const int32_t* g_idx, int groupsize, void* out, int K, int N,
                                 hipStream_t stream) {
    const long total = (long)(K / 8) * (N / 8);
    const int threads = 256;
    const long blocks = (total + threads - 1) / threads;
    hipLaunchKernelGGL(q4::dequant_kernel, dim3((unsigned)blocks), dim3(threads), 0, stream,
                       reinterpret_cast<const uint32_t*>(qweight), reinterpret_cast<const uint32_t*>(qzeros),
                       reinterpret_cast<const q4::half_t*>(scales), g_idx, groupsize,
                       reinterpret_cast<q4::half_t*>(out), K, N);
    return hipGetLastError() == hipSuccess ? 0 : -4;
}
