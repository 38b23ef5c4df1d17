// Rank-R helper products of the LoRA adapter around the fused 4-bit GEMMs (HBM-bound: each reads
// one [M, C] activation / gradient matrix exactly once).
//
//   down:  out fp16 [M, R]   = in fp16 [M, C] @ W^T          xa = x @ A^T,  dyb = dy @ B
//   grad:  out fp32 [R, C]^  = alpha * P^T fp16 [R, M] @ in   dA = s * dyb^T @ x,  dB^T = s * xa^T @ dy
//
// (^ written through strides, so dB lands directly in lora_B.weight's [N, R] layout.)
// Together with the adapter step inside the GEMMs they replace what torch autograd does over
// lora_B(lora_A(x)) * scaling in the reference (src/alpaca_lora_4bit/models.py:58-66).
// W is read in place with strides and in its own dtype (fp32 or fp16): no cast or transpose
// kernels around the adapter.
#include "q4_common.hpp"

namespace q4 {

constexpr int kFracBits = 24;
constexpr long long kBias = 1ll << 47;
constexpr float kClamp = 4194304.0f;

__device__ __forceinline__ half8_t load_w8(const void* w, int is_f32, size_t idx0, int stride_c) {
    // eight consecutive-c elements W[j, c0 .. c0+7] as fp16
    half8_t r;
    if (is_f32) {
        const float* p = reinterpret_cast<const float*>(w) + idx0;
        if (stride_c == 1 && (idx0 & 3) == 0) {
            const float4_t a = *reinterpret_cast<const float4_t*>(p), b = *reinterpret_cast<const float4_t*>(p + 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) { r[e] = (half_t)a[e]; r[4 + e] = (half_t)b[e]; }
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) r[e] = (half_t)p[(size_t)e * stride_c];
        }
    } else {
        const half_t* p = reinterpret_cast<const half_t*>(w) + idx0;
        if (stride_c == 1 && (idx0 & 7) == 0) {
            r = *reinterpret_cast<const half8_t*>(p);
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) r[e] = p[(size_t)e * stride_c];
        }
    }
    return r;
}

// ---- down projection -------------------------------------------------------------------
// Workgroup = 8 wavefronts on 16 rows; wavefront w multiplies the C/8-wide slice w of those rows
// with v_mfma_f32_16x16x32_f16 (A operand = 16 rows x 32 columns of `in`, B operand = the same 32
// columns of up to 16 rows of W), partial 16 x 16 results are added through LDS.
// R <= 64 is handled as ceil(R/16) column blocks.
template <int RB>   // number of 16-wide blocks of R
__global__ __launch_bounds__(512) void lora_down_kernel(const half_t* __restrict__ in, const void* __restrict__ w,
                                                        int w_sr, int w_sc, int w_is_f32, half_t* __restrict__ out,
                                                        int M, int C, int R) {
    __shared__ float red[8][RB][256];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kk = lane >> 4, c = lane & 15;
    const int m0 = blockIdx.x * 16;
    const int row = min(m0 + c, M - 1);
    const int steps = C / 32;                                   // C is a multiple of 32
    const int s_begin = (steps * wave) / 8, s_end = (steps * (wave + 1)) / 8;
    float4_t acc[RB];
#pragma unroll
    for (int b = 0; b < RB; ++b) acc[b] = float4_t{0.f, 0.f, 0.f, 0.f};
    const half_t* ip = in + (size_t)row * C + 8 * kk;
    constexpr int UN = RB == 1 ? 8 : 4;                        // steps whose loads are issued together
    for (int s0 = s_begin; s0 < s_end; s0 += UN) {
        half8_t av[UN], bv[UN][RB];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int s = min(s0 + u, s_end - 1);               // tail steps repeat the last one and are skipped below
            av[u] = *reinterpret_cast<const half8_t*>(ip + 32 * s);
#pragma unroll
            for (int b = 0; b < RB; ++b) {
                const int j = 16 * b + c;
#pragma unroll
                for (int e = 0; e < 8; ++e) bv[u][b][e] = (half_t)0.f;
                if (j < R) bv[u][b] = load_w8(w, w_is_f32, (size_t)j * w_sr + (size_t)(32 * s + 8 * kk) * w_sc, w_sc);
            }
        }
#pragma unroll
        for (int u = 0; u < UN; ++u)
            if (s0 + u < s_end)
#pragma unroll
                for (int b = 0; b < RB; ++b)
                    acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[u], bv[u][b], acc[b], 0, 0, 0);
    }
    // acc[b][r]: row 4*kk + r, column 16*b + c
#pragma unroll
    for (int b = 0; b < RB; ++b)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[wave][b][(4 * kk + r) * 16 + c] = acc[b][r];
    __syncthreads();
    for (int e = threadIdx.x; e < RB * 256; e += 512) {
        const int b = e >> 8, i = e & 255;
        float v = 0.f;
#pragma unroll
        for (int wv = 0; wv < 8; ++wv) v += red[wv][b][i];
        const int m = m0 + (i >> 4), j = 16 * b + (i & 15);
        if (m < M && j < R) out[(size_t)m * R + j] = (half_t)v;
    }
}

// ---- gradient of an adapter matrix -------------------------------------------------------
// out[j, c] = alpha * sum_m P[m, j] * in[m, c].  A thread owns CPT = 64/R8 adjacent columns
// (R8 = R rounded up to 8... here R in {8, 16}: 8 or 4 columns) and R x CPT fp32 accumulators; the
// 8 wavefronts of a workgroup share a block of 64*CPT columns and split its rows; gridDim.y
// workgroups share a column block.  Rows of P reach the lanes as LDS broadcasts.  The reduction
// over wavefronts goes through LDS, the one over workgroups through one 64-bit fixed-point
// atomic per output element with an arrival count in the top byte (order-independent, hence
// bit-reproducible; the last arrival converts, scales and stores, and zeroes the workspace).
template <int R>
__global__ __launch_bounds__(512) void lora_grad_kernel(const half_t* __restrict__ P, const half_t* __restrict__ in,
                                                        float* __restrict__ out, int o_sr, int o_sc, float alpha,
                                                        int M, int C, int rows_per_wg,
                                                        unsigned long long* __restrict__ acc64) {
    constexpr int CPT = 64 / R;                  // columns per thread: 8 (R = 8) or 4 (R = 16)
    constexpr int NACC = R * CPT;                // 64
    __shared__ float red[8][NACC][64];           // 128 KB
    __shared__ __attribute__((aligned(16))) half_t ptile[8][16][R];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c0 = (blockIdx.x * 64 + lane) * CPT;
    const bool col_ok = c0 < C;                  // C is a multiple of 8, so a thread's columns are all in or all out
    const int m_begin = blockIdx.y * rows_per_wg + wave * (rows_per_wg / 8);
    const int m_end = min(m_begin + rows_per_wg / 8, M);
    float acc[R][CPT];
#pragma unroll
    for (int j = 0; j < R; ++j)
#pragma unroll
        for (int e = 0; e < CPT; ++e) acc[j][e] = 0.f;

    for (int mb = m_begin; mb < m_end; mb += 16) {
        // stage 16 rows of P for this wavefront (wavefront-private region, LDS ops of a wave are ordered)
        const int nrow = min(16, m_end - mb);
        for (int i = lane; i < 16 * R; i += 64) {
            const int rr = i / R, j = i - rr * R;
            ptile[wave][rr][j] = rr < nrow ? P[(size_t)(mb + rr) * R + j] : (half_t)0.f;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // all 16 row loads of `in` first, then the arithmetic
        half_t xin[16][CPT];
#pragma unroll
        for (int rr = 0; rr < 16; ++rr) {
            const int m = min(mb + rr, M - 1);
            if (col_ok) {
                if constexpr (CPT == 8) {
                    const half8_t v = *reinterpret_cast<const half8_t*>(in + (size_t)m * C + c0);
#pragma unroll
                    for (int e = 0; e < 8; ++e) xin[rr][e] = v[e];
                } else {
                    const half4_t v = *reinterpret_cast<const half4_t*>(in + (size_t)m * C + c0);
#pragma unroll
                    for (int e = 0; e < 4; ++e) xin[rr][e] = v[e];
                }
            } else {
#pragma unroll
                for (int e = 0; e < CPT; ++e) xin[rr][e] = (half_t)0.f;
            }
        }
#pragma unroll
        for (int rr = 0; rr < 16; ++rr) {
            half_t p[R];
#pragma unroll
            for (int j = 0; j < R; j += 8) {
                const half8_t pv = *reinterpret_cast<const half8_t*>(&ptile[wave][rr][j]);
#pragma unroll
                for (int e = 0; e < 8; ++e) p[j + e] = pv[e];
            }
#pragma unroll
            for (int j = 0; j < R; ++j)
#pragma unroll
                for (int e = 0; e < CPT; ++e) acc[j][e] += (float)p[j] * (float)xin[rr][e];
        }
        __builtin_amdgcn_wave_barrier();
    }
#pragma unroll
    for (int j = 0; j < R; ++j)
#pragma unroll
        for (int e = 0; e < CPT; ++e) red[wave][j * CPT + e][lane] = acc[j][e];
    __syncthreads();
    const int S = gridDim.y;
    for (int o = threadIdx.x; o < NACC * 64; o += 512) {
        const int a = o >> 6, ln = o & 63;
        float v = 0.f;
#pragma unroll
        for (int wv = 0; wv < 8; ++wv) v += red[wv][a][ln];
        const int j = a / CPT, cc = (blockIdx.x * 64 + ln) * CPT + (a - j * CPT);
        if (cc >= C) continue;
        float* op = out + (size_t)j * o_sr + (size_t)cc * o_sc;
        if (S == 1) {
            *op = alpha * v;
        } else {
            v = fminf(fmaxf(v, -kClamp), kClamp);
            const long long fx = __float2ll_rn(v * (float)(1 << kFracBits));
            const unsigned long long add = (1ull << 56) + (unsigned long long)(fx + kBias);
            unsigned long long* ap = acc64 + (size_t)j * C + cc;
            const unsigned long long old = __hip_atomic_fetch_add(ap, add, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if ((old >> 56) == (unsigned long long)(S - 1)) {
                const long long tot = (long long)((old + add) & ((1ull << 56) - 1)) - (long long)S * kBias;
                *op = alpha * (float)((double)tot * (1.0 / (double)(1 << kFracBits)));
                __hip_atomic_store(ap, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
}

}  // namespace q4

extern "C" int q4_launch_lora_down(const void* in, const void* w, int w_sr, int w_sc, int w_is_f32, void* out,
                                   int M, int C, int R, hipStream_t stream) {
    using namespace q4;
    const dim3 grid((M + 15) / 16), block(512);
    const half_t* ip = reinterpret_cast<const half_t*>(in);
    half_t* op = reinterpret_cast<half_t*>(out);
    switch ((R + 15) / 16) {
        case 1: hipLaunchKernelGGL(lora_down_kernel<1>, grid, block, 0, stream, ip, w, w_sr, w_sc, w_is_f32, op, M, C, R); break;
        case 2: hipLaunchKernelGGL(lora_down_kernel<2>, grid, block, 0, stream, ip, w, w_sr, w_sc, w_is_f32, op, M, C, R); break;
        case 3: hipLaunchKernelGGL(lora_down_kernel<3>, grid, block, 0, stream, ip, w, w_sr, w_sc, w_is_f32, op, M, C, R); break;
        default: hipLaunchKernelGGL(lora_down_kernel<4>, grid, block, 0, stream, ip, w, w_sr, w_sc, w_is_f32, op, M, C, R); break;
    }
    return hipGetLastError() == hipSuccess ? 0 : -4;
}

extern "C" int q4_launch_lora_grad(const void* P, const void* in, float* out, int o_sr, int o_sc, float alpha,
                                   int M, int C, int R, void* workspace, hipStream_t stream) {
    using namespace q4;
    const int cpt = 64 / R;
    const int col_blocks = (C + 64 * cpt - 1) / (64 * cpt);
    // rows per workgroup: a multiple of 128 (8 wavefronts x 16 rows); the LDS footprint allows one
    // workgroup per CU, so aim at about one workgroup for each of the 256 CUs
    int splits = (256 + col_blocks - 1) / col_blocks;
    int rows_per_wg = ((M + splits - 1) / splits + 127) / 128 * 128;
    if (rows_per_wg < 128) rows_per_wg = 128;
    splits = (M + rows_per_wg - 1) / rows_per_wg;
    if (splits > 255) { rows_per_wg = ((M + 254) / 255 + 127) / 128 * 128; splits = (M + rows_per_wg - 1) / rows_per_wg; }
    const dim3 grid(col_blocks, splits), block(512);
    const half_t* pp = reinterpret_cast<const half_t*>(P);
    const half_t* ip = reinterpret_cast<const half_t*>(in);
    unsigned long long* ws = reinterpret_cast<unsigned long long*>(workspace);
    if (R == 8) hipLaunchKernelGGL(lora_grad_kernel<8>, grid, block, 0, stream, pp, ip, out, o_sr, o_sc, alpha, M, C, rows_per_wg, ws);
    else hipLaunchKernelGGL(lora_grad_kernel<16>, grid, block, 0, stream, pp, ip, out, o_sr, o_sc, alpha, M, C, rows_per_wg, ws);
    return hipGetLastError() == hipSuccess ? 0 : -4;
}
