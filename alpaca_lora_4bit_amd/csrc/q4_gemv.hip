// Decode GEMV / skinny GEMM for 1 <= M <= 16:  y[M,N] = x[M,K] @ W   (HBM-bound).
//
// Work split.  One wavefront owns a strip of 64 columns and a chunk of 32*NSTEP rows.  Lane l
// (kk = l / 16, c = l % 16) reads, per step of 32 rows, ONE 128-bit vector
// qweight[row/8 + kk, n0 + 4c .. 4c+3]: four packed words, i.e. 8 consecutive rows of four
// adjacent columns.  A packed word is exactly the 8-deep k-slice that lane l feeds to
// v_mfma_f32_16x16x32_f16 as its B operand, so the four words go to four MFMAs whose column
// index i stands for column n0 + 4i + j (j = 0..3).  The A operand is x (row m = l % 16, the
// same 8 k values; rows >= M are zero), so all M <= 16 activation rows ride along for free and
// the weights are read from HBM once.  All NSTEP weight vectors of a lane are requested before
// the first is used: with ~90 KB of weights per CU the kernel is a single burst of loads.
//
// Sequential groups (no act-order).  The B operand holds the raw codes as fp16 (1024 + q)
// and a fifth MFMA with an all-ones B operand yields X = sum_k x over the same rows, so per
// group only   y += s * (acc - (1025 + z) * X)   is evaluated (fp32) instead of one
// multiply-subtract per weight.  Mathematically equal to sum_k x*(s*q - s*(z+1))
// (src/alpaca_lora_4bit/quant_cuda/quant_cuda_kernel.cu:1026-1037); not bit-identical to it,
// nor is the reference to itself (fp16 partial sums and atomicAdd order, :1037,1040).
//
// Act-order.  Rows of one word can belong to 8 different groups, so the B operand is built
// from explicitly dequantized weights with (scale, zero) gathered through g_idx per row
// (the convention of VecQuant4MatMulKernel, quant_cuda_kernel.cu:513-520).
//
// Split-K.  gridDim.y chunks of K produce fp32 partials in the workspace; the last
// workgroup to arrive for a column strip (agent-scope counter) adds them in chunk order, so
// the result does not depend on scheduling, and resets the counter for the next call.
#include "q4_common.hpp"

namespace q4 {

constexpr int kWavesPerBlock = 4;
constexpr int kColsPerWave = 64;

struct GemvArgs {
    const half_t* x;
    const uint32_t* qweight;
    const uint32_t* qzeros;
    const half_t* scales;
    const int32_t* g_idx;
    int groupsize;
    half_t* y;
    int accumulate;
    int M, K, N;
    float* partials;      // [S, M, N]
    uint32_t* counters;   // [gridDim.x]
};

__device__ __forceinline__ half8_t make_half8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    uint4_t v = {a, b, c, d};
    return __builtin_bit_cast(half8_t, v);
}

// Writes the wave's fp32 results: straight to y when there is one chunk, else partials +
// last-arriver reduction.  yacc[j][r] belongs to row 4*kk + r, column n0 + 4c + j.
__device__ __forceinline__ void gemv_finish(const GemvArgs& a, const float4_t yacc[4], bool wave_active,
                                            int n0, int kk, int c) {
    const int S = gridDim.y;
    const int col = n0 + 4 * c;
    if (S == 1) {
        if (wave_active) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = 4 * kk + r;
                if (m < a.M) {
                    half_t* yp = a.y + (size_t)m * a.N + col;
                    float v[4] = {yacc[0][r], yacc[1][r], yacc[2][r], yacc[3][r]};
                    if (a.accumulate) {
                        const half4_t old = *reinterpret_cast<const half4_t*>(yp);
#pragma unroll
                        for (int j = 0; j < 4; ++j) v[j] += (float)old[j];
                    }
                    half4_t o = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
                    *reinterpret_cast<half4_t*>(yp) = o;
                }
            }
        }
        return;
    }
    if (wave_active) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int m = 4 * kk + r;
            if (m < a.M) {
                float4_t v = {yacc[0][r], yacc[1][r], yacc[2][r], yacc[3][r]};
                *reinterpret_cast<float4_t*>(a.partials + ((size_t)blockIdx.y * a.M + m) * a.N + col) = v;
            }
        }
    }
    __shared__ int s_last;
    __threadfence();                       // release the partials at agent scope
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t old = __hip_atomic_fetch_add(a.counters + blockIdx.x, 1u, __ATOMIC_ACQ_REL,
                                                    __HIP_MEMORY_SCOPE_AGENT);
        s_last = (old == (uint32_t)(S - 1));
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();                       // acquire the other workgroups' partials
    if (wave_active) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int m = 4 * kk + r;
            if (m < a.M) {
                float4_t sum = {0.f, 0.f, 0.f, 0.f};
                const float* pp = a.partials + (size_t)m * a.N + col;
                const size_t stride = (size_t)a.M * a.N;
                for (int s = 0; s < S; ++s)
                    sum += *reinterpret_cast<const float4_t*>(pp + (size_t)s * stride);
                half_t* yp = a.y + (size_t)m * a.N + col;
                if (a.accumulate) {
                    const half4_t old = *reinterpret_cast<const half4_t*>(yp);
#pragma unroll
                    for (int j = 0; j < 4; ++j) sum[j] += (float)old[j];
                }
                half4_t o = {(half_t)sum[0], (half_t)sum[1], (half_t)sum[2], (half_t)sum[3]};
                *reinterpret_cast<half4_t*>(yp) = o;
            }
        }
    }
    if (threadIdx.x == 0) a.counters[blockIdx.x] = 0u;   // leave the workspace zeroed
}

// ------------------------------------------------------------------ sequential groups
template <int NSTEP>
__global__ __launch_bounds__(64 * kWavesPerBlock) void gemv_seq_kernel(GemvArgs a) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int kk = lane >> 4, c = lane & 15;
    const int n0 = (blockIdx.x * kWavesPerBlock + wave) * kColsPerWave;
    const bool wave_active = n0 < a.N;
    const int k0 = blockIdx.y * (32 * NSTEP);

    float4_t yacc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) yacc[j] = float4_t{0.f, 0.f, 0.f, 0.f};

    if (wave_active) {
        const int ncol8 = a.N >> 3;
        // ---- issue every load of this chunk up front
        uint4_t wv[NSTEP], xv[NSTEP];
#pragma unroll
        for (int t = 0; t < NSTEP; ++t) {
            const int ks = k0 + 32 * t;
            wv[t] = uint4_t{0u, 0u, 0u, 0u};
            xv[t] = uint4_t{0u, 0u, 0u, 0u};
            if (ks < a.K) {
                wv[t] = *reinterpret_cast<const uint4_t*>(a.qweight + (size_t)((ks >> 3) + kk) * a.N + n0 + 4 * c);
                if (c < a.M)
                    xv[t] = *reinterpret_cast<const uint4_t*>(a.x + (size_t)c * a.K + ks + 8 * kk);
            }
        }
        const int kend = min(k0 + 32 * NSTEP, a.K);
        const int g_first = k0 / a.groupsize;
        const int g_last = (kend - 1) / a.groupsize;
        // scale / zero of the first two groups travel with the burst; later ones on demand
        uint2_t sv[2];
        uint32_t zv[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int g = min(g_first + i, g_last);
            sv[i] = *reinterpret_cast<const uint2_t*>(a.scales + (size_t)g * a.N + n0 + 4 * c);
            zv[i] = a.qzeros[(size_t)g * ncol8 + ((n0 + 4 * c) >> 3)];
        }

        const half8_t ones = make_half8(0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u);
        float4_t acc[4], accx;
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = float4_t{0.f, 0.f, 0.f, 0.f};
        accx = float4_t{0.f, 0.f, 0.f, 0.f};

        auto flush = [&](int g) {
            uint2_t s4;
            uint32_t zw;
            const int gi = g - g_first;
            if (gi == 0) { s4 = sv[0]; zw = zv[0]; }
            else if (gi == 1) { s4 = sv[1]; zw = zv[1]; }
            else {
                s4 = *reinterpret_cast<const uint2_t*>(a.scales + (size_t)g * a.N + n0 + 4 * c);
                zw = a.qzeros[(size_t)g * ncol8 + ((n0 + 4 * c) >> 3)];
            }
            zw >>= (c & 1) * 16;
            const half2_t s01 = as_half2(s4.x), s23 = as_half2(s4.y);
            const float sf[4] = {(float)s01[0], (float)s01[1], (float)s23[0], (float)s23[1]};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float zf = (float)(((zw >> (4 * j)) & 0xFu) + 1025u);
#pragma unroll
                for (int r = 0; r < 4; ++r) yacc[j][r] += sf[j] * (acc[j][r] - zf * accx[r]);
                acc[j] = float4_t{0.f, 0.f, 0.f, 0.f};
            }
            accx = float4_t{0.f, 0.f, 0.f, 0.f};
        };

        int gcur = g_first;
#pragma unroll
        for (int t = 0; t < NSTEP; ++t) {
            const int ks = k0 + 32 * t;
            if (ks < a.K) {
                const int g = ks / a.groupsize;
                if (g != gcur) { flush(gcur); gcur = g; }
                // A operand in the order the cheap nibble split produces: (e0,e4)(e1,e5)(e2,e6)(e3,e7)
                const half8_t av = make_half8(__builtin_amdgcn_perm(xv[t].z, xv[t].x, 0x05040100u),
                                              __builtin_amdgcn_perm(xv[t].z, xv[t].x, 0x07060302u),
                                              __builtin_amdgcn_perm(xv[t].w, xv[t].y, 0x05040100u),
                                              __builtin_amdgcn_perm(xv[t].w, xv[t].y, 0x07060302u));
                const uint32_t w[4] = {wv[t].x, wv[t].y, wv[t].z, wv[t].w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const half8_t bv = make_half8((w[j] & 0x000F000Fu) | kMagic, ((w[j] >> 4) & 0x000F000Fu) | kMagic,
                                                  ((w[j] >> 8) & 0x000F000Fu) | kMagic, ((w[j] >> 12) & 0x000F000Fu) | kMagic);
                    acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, bv, acc[j], 0, 0, 0);
                }
                accx = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, ones, accx, 0, 0, 0);
            }
        }
        flush(gcur);
    }
    gemv_finish(a, yacc, wave_active, n0, kk, c);
}

// ------------------------------------------------------------------ act-order (per-row groups)
template <int NSTEP>
__global__ __launch_bounds__(64 * kWavesPerBlock) void gemv_gidx_kernel(GemvArgs a) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int kk = lane >> 4, c = lane & 15;
    const int n0 = (blockIdx.x * kWavesPerBlock + wave) * kColsPerWave;
    const bool wave_active = n0 < a.N;
    const int k0 = blockIdx.y * (32 * NSTEP);

    float4_t yacc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) yacc[j] = float4_t{0.f, 0.f, 0.f, 0.f};

    if (wave_active) {
        const int ncol8 = a.N >> 3;
        const int col = n0 + 4 * c;
        const int zshift = (c & 1) * 16;
        uint4_t wv[NSTEP], xv[NSTEP];
#pragma unroll
        for (int t = 0; t < NSTEP; ++t) {
            const int ks = k0 + 32 * t;
            wv[t] = uint4_t{0u, 0u, 0u, 0u};
            xv[t] = uint4_t{0u, 0u, 0u, 0u};
            if (ks < a.K) {
                wv[t] = *reinterpret_cast<const uint4_t*>(a.qweight + (size_t)((ks >> 3) + kk) * a.N + col);
                if (c < a.M)
                    xv[t] = *reinterpret_cast<const uint4_t*>(a.x + (size_t)c * a.K + ks + 8 * kk);
            }
        }
#pragma unroll
        for (int t = 0; t < NSTEP; ++t) {
            const int ks = k0 + 32 * t;
            if (ks < a.K) {
                const int kb = ks + 8 * kk;
                const uint4_t ga = *reinterpret_cast<const uint4_t*>(a.g_idx + kb);
                const uint4_t gb = *reinterpret_cast<const uint4_t*>(a.g_idx + kb + 4);
                const uint32_t g[8] = {ga.x, ga.y, ga.z, ga.w, gb.x, gb.y, gb.z, gb.w};
                uint2_t s4[8];
                uint32_t zw[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    s4[e] = *reinterpret_cast<const uint2_t*>(a.scales + (size_t)g[e] * a.N + col);
                    zw[e] = a.qzeros[(size_t)g[e] * ncol8 + (col >> 3)] >> zshift;
                }
                const half8_t av = make_half8(xv[t].x, xv[t].y, xv[t].z, xv[t].w);
                const uint32_t w[4] = {wv[t].x, wv[t].y, wv[t].z, wv[t].w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    half2_t q2[4];
                    unpack8_natural(w[j], q2);
                    uint32_t b[4];
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        const int e0 = 2 * p, e1 = 2 * p + 1;
                        const uint32_t sa = (j < 2) ? s4[e0].x : s4[e0].y;
                        const uint32_t sb = (j < 2) ? s4[e1].x : s4[e1].y;
                        // (scale of row e0, scale of row e1) for column j
                        const half2_t s2 = as_half2((j & 1) ? __builtin_amdgcn_perm(sb, sa, 0x07060302u)
                                                            : __builtin_amdgcn_perm(sb, sa, 0x05040100u));
                        const half2_t z2 = zero_term(s2, (zw[e0] >> (4 * j)) & 0xFu, (zw[e1] >> (4 * j)) & 0xFu);
                        b[p] = as_u32(dequant_pair(q2[p], s2, z2));
                    }
                    yacc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, make_half8(b[0], b[1], b[2], b[3]), yacc[j], 0, 0, 0);
                }
            }
        }
    }
    gemv_finish(a, yacc, wave_active, n0, kk, c);
}

}  // namespace q4

// Chunk length (in 32-row steps) so that the grid has enough wavefronts to cover the chip
// while the fp32 partials stay a small fraction of the weight bytes.
static int pick_nstep(int M, int K, int N) {
    const long strips = N / q4::kColsPerWave;
    const long steps = (K + 31) / 32;
    for (int nstep : {16, 8, 4}) {
        const long waves = strips * ((steps + nstep - 1) / nstep);
        if (waves >= 2048 || nstep == 4) {
            if (M > 4 && nstep < 8) return 8;      // keep the partials small for wide batches
            return nstep;
        }
    }
    return 4;
}

extern "C" size_t q4_gemv_workspace_bytes(int M, int K, int N) {
    if (M < 1 || K < 1 || N < 1) return 0;
    const size_t S = (size_t)(K + 127) / 128;                     // upper bound on chunks
    const size_t counters = 4096;                                   // bytes, >= 4 * ceil(N/256) for N <= 262144
    return counters + S * (size_t)M * (size_t)N * sizeof(float);
}

extern "C" int q4_launch_gemv(const void* x, const int32_t* qweight, const int32_t* qzeros, const void* scales,
                              const int32_t* g_idx, int groupsize, void* y, int accumulate,
                              int M, int K, int N, void* workspace, hipStream_t stream) {
    using namespace q4;
    GemvArgs a;
    a.x = reinterpret_cast<const half_t*>(x);
    a.qweight = reinterpret_cast<const uint32_t*>(qweight);
    a.qzeros = reinterpret_cast<const uint32_t*>(qzeros);
    a.scales = reinterpret_cast<const half_t*>(scales);
    a.g_idx = g_idx;
    a.groupsize = groupsize;
    a.y = reinterpret_cast<half_t*>(y);
    a.accumulate = accumulate;
    a.M = M; a.K = K; a.N = N;
    a.counters = reinterpret_cast<uint32_t*>(workspace);
    a.partials = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + 4096);

    const int nstep = pick_nstep(M, K, N);
    const int steps = (K + 31) / 32;
    const dim3 grid((N / kColsPerWave + kWavesPerBlock - 1) / kWavesPerBlock, (steps + nstep - 1) / nstep);
    const dim3 block(64 * kWavesPerBlock);
    const bool seq = (g_idx == nullptr);
#define Q4_LAUNCH(NS)                                                                     \
    do {                                                                                  \
        if (seq) hipLaunchKernelGGL(gemv_seq_kernel<NS>, grid, block, 0, stream, a);      \
        else hipLaunchKernelGGL(gemv_gidx_kernel<NS>, grid, block, 0, stream, a);         \
    } while (0)
    if (nstep == 16) Q4_LAUNCH(16);
    else if (nstep == 8) Q4_LAUNCH(8);
    else Q4_LAUNCH(4);
#undef Q4_LAUNCH
    return hipGetLastError() == hipSuccess ? 0 : -4;
}
