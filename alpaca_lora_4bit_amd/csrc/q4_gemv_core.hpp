// Core of the weight-streaming GEMV for 1..16 activation rows on sequential groups: launch arguments, the per-wavefront
// chunk (loads, operand build, MFMAs, group epilogue) and the reduction over K (LDS inside a workgroup, one 64-bit
// fixed-point atomic per output element across workgroups).  Shared by q4_gemv.hip (single layers, grouped layers) and
// q4_mlp.hip (gate|up -> activation -> down in one launch).  The scheme is described at the top of q4_gemv.hip.
#pragma once
#include "q4_common.hpp"
#include <stdlib.h>

namespace q4 {

constexpr int kColsPerWave = 64;
constexpr int kFracBits = 24;
constexpr long long kBias = 1ll << 47;
constexpr float kClamp = 4194304.0f;          // 2^22: |partial| beyond this saturates (fp16 max is 65504)

struct GemvArgs {
    const half_t* x;
    const uint32_t* qweight;
    const uint32_t* qzeros;
    const half_t* scales;
    const int32_t* g_idx;
    int groupsize;
    half_t* y;
    int accumulate;
    int M, K, N, G;
    unsigned long long* acc64;   // [M, N], zero between calls
    const int32_t* perm;         // gemv_seq_perm_kernel only: original index of every (sorted) reduction row
    const half_t* v1_zeros;      // v1 layout only: fp16 zero value per column
};

__device__ __forceinline__ half8_t make_half8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    uint4_t v = {a, b, c, d};
    return __builtin_bit_cast(half8_t, v);
}

// Finishes EB outputs per thread (e0, e0 + blockDim.x, ...): all LDS reads of the batch are issued before
// the first sum needs them and all atomics of the batch are in flight before the first reply is looked at,
// so a thread pays one LDS latency and one atomic round trip per batch, not per term.
//
// `hand` (null for a plain product): the complete output is ALSO published as one 32-bit word per element, the fp16 bits
// in the low half and `tag` in the high half, with a device-scope atomic store.  A consumer in the same launch that
// reads a word carrying the launch's tag holds the finished value: value and flag travel in one atomic object, so
// the hand-over needs no fence (see q4_mlp.hip).  In that mode y may be null.
template <int EB>
__device__ __forceinline__ void gemv_finish_batch(const GemvArgs& a, const float* red, int e0, int total, int n0,
                                                  int nwaves, int S, uint32_t* hand, uint32_t tag) {
    const int M = a.M;
    float v[EB];
#pragma unroll
    for (int i = 0; i < EB; ++i) {
        const int e = min(e0 + i * (int)blockDim.x, total - 1);
        float t = 0.f;
        int w = 0;
        for (; w + 8 <= nwaves; w += 8) {
            float p[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) p[u] = red[(((w + u) * M) << 6) + e];
            t += ((p[0] + p[1]) + (p[2] + p[3])) + ((p[4] + p[5]) + (p[6] + p[7]));
        }
        for (; w < nwaves; ++w) t += red[((w * M) << 6) + e];
        v[i] = t;
    }
    if (S == 1) {
#pragma unroll
        for (int i = 0; i < EB; ++i) {
            const int e = e0 + i * blockDim.x;
            if (e < total) {
                const size_t at = (size_t)(e >> 6) * a.N + n0 + (e & 63);
                float out = v[i];
                if (a.accumulate) out += (float)a.y[at];
                const half_t h = (half_t)out;
                if (!hand || a.y) a.y[at] = h;
                if (hand)
                    __hip_atomic_store(hand + at, (uint32_t)__builtin_bit_cast(unsigned short, h) | (tag << 16),
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        return;
    }
    unsigned long long old[EB], add[EB];
#pragma unroll
    for (int i = 0; i < EB; ++i) {
        const int e = e0 + i * blockDim.x;
        const float c = fminf(fmaxf(v[i], -kClamp), kClamp);
        const long long fx = __float2ll_rn(c * (float)(1 << kFracBits));
        add[i] = (1ull << 56) + (unsigned long long)(fx + kBias);
        old[i] = 0;
        if (e < total)
            old[i] = __hip_atomic_fetch_add(a.acc64 + (size_t)(e >> 6) * a.N + n0 + (e & 63), add[i],
                                            __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
#pragma unroll
    for (int i = 0; i < EB; ++i) {
        const int e = e0 + i * blockDim.x;
        if (e < total && (old[i] >> 56) == (unsigned long long)(S - 1)) {      // last of the S workgroups of the strip
            const size_t at = (size_t)(e >> 6) * a.N + n0 + (e & 63);
            const long long tot = (long long)((old[i] + add[i]) & ((1ull << 56) - 1)) - (long long)S * kBias;
            float out = (float)((double)tot * (1.0 / (double)(1 << kFracBits)));
            if (a.accumulate) out += (float)a.y[at];
            const half_t h = (half_t)out;
            if (!hand || a.y) a.y[at] = h;
            if (hand)
                __hip_atomic_store(hand + at, (uint32_t)__builtin_bit_cast(unsigned short, h) | (tag << 16),
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(a.acc64 + at, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// yacc[j][r] of this lane belongs to row 4*kk + r, column n0 + 4c + j.
// S = number of workgroups that share the strip (the K splits).
__device__ __forceinline__ void gemv_finish(const GemvArgs& a, const float4_t yacc[4], int n0, int wave, int nwaves,
                                            int kk, int c, int S, uint32_t* hand = nullptr,
                                            const uint32_t* tag_lds = nullptr) {
    extern __shared__ float red[];               // [nwaves][M][64]
    const int M = a.M;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int m = 4 * kk + r;
        if (m < M)
            *reinterpret_cast<float4_t*>(red + ((wave * M + m) << 6) + 4 * c) =
                float4_t{yacc[0][r], yacc[1][r], yacc[2][r], yacc[3][r]};
    }
    __syncthreads();
    const uint32_t tag = hand ? *tag_lds : 0u;   // written to LDS by one thread of the workgroup before the barrier
    const int total = M * 64;
    if (total <= (int)blockDim.x) {              // at most one output per thread (uniform)
        if ((int)threadIdx.x < total) gemv_finish_batch<1>(a, red, threadIdx.x, total, n0, nwaves, S, hand, tag);
    } else {
        for (int e0 = threadIdx.x; e0 < total; e0 += 2 * blockDim.x) gemv_finish_batch<2>(a, red, e0, total, n0, nwaves, S, hand, tag);
    }
}

// ------------------------------------------------------------------ sequential groups
// GSTEPS = steps of 32 rows per quantization group (1, 2, 4, 8; NSTEP % GSTEPS == 0), or
// 0 when a whole chunk lies inside one group (groupsize % (32*NSTEP) == 0).
// V1: the older layout with one fp16 scale and one fp16 zero VALUE per column (no groups, no zero codes):
// W = s*q - zero (quant_cuda_kernel.cu:1076-1097), so y = s * sum(x*q) - zero * sum(x).
template <int NSTEP, int GSTEPS, bool V1 = false>
struct SeqChunk {
    static constexpr int NG = GSTEPS == 0 ? 1 : NSTEP / GSTEPS;
    static constexpr int GS = GSTEPS == 0 ? NSTEP : GSTEPS;
    static_assert(!V1 || GSTEPS == 0, "the v1 layout has a single group");
    uint2_t sv[NG];
    uint32_t zv[NG];
    uint2_t zh;                                   // V1: four fp16 zeros
    uint4_t wv[NSTEP], xv[NSTEP];

    // scale / zero of every group of the chunk first: they are consumed last but must not sit behind the
    // weights in the in-order return queue.  The packed words are read exactly once per product: streaming
    // loads, so they do not displace the activations and scales that every strip shares from the caches.
    __device__ __forceinline__ void load_weights(const GemvArgs& a, int k0, int col, int kk) {
        if constexpr (V1) {
            sv[0] = *reinterpret_cast<const uint2_t*>(a.scales + col);
            zh = *reinterpret_cast<const uint2_t*>(a.v1_zeros + col);
        } else {
            const int ncol8 = a.N >> 3;
            const int g0 = k0 / a.groupsize;
#pragma unroll
            for (int i = 0; i < NG; ++i) {
                sv[i] = *reinterpret_cast<const uint2_t*>(a.scales + (size_t)(g0 + i) * a.N + col);
                zv[i] = a.qzeros[(size_t)(g0 + i) * ncol8 + (col >> 3)];
            }
        }
        const rsrc_t rw = make_rsrc(a.qweight, (unsigned)((size_t)(a.K >> 3) * a.N * 4));
        const int vw = (((k0 >> 3) + kk) * a.N + col) * 4;
#pragma unroll
        for (int t = 0; t < NSTEP; ++t) wv[t] = buf_load128_stream(rw, vw, 16 * t * a.N);
    }

    // The same without a branch around it: a wavefront past the end of K (wave-uniform `live` false) fetches
    // from an offset beyond every buffer, which returns zeros without traffic.
    __device__ __forceinline__ void load_weights_branch_free(const GemvArgs& a, int k0, int col, int kk, bool live) {
        constexpr int kFar = 0x70000000;
        const int ncol8 = a.N >> 3;
        const int g0 = live ? k0 / a.groupsize : 0;
        const int off = live ? 0 : kFar;
        const rsrc_t rs = make_rsrc(a.scales, (unsigned)((size_t)a.G * a.N * 2));
        const rsrc_t rz = make_rsrc(a.qzeros, (unsigned)((size_t)a.G * ncol8 * 4));
#pragma unroll
        for (int i = 0; i < NG; ++i) {
            sv[i] = buf_load64(rs, ((g0 + i) * a.N + col) * 2, off);
            zv[i] = buf_load32(rz, ((g0 + i) * ncol8 + (col >> 3)) * 4, off);
        }
        const rsrc_t rw = make_rsrc(a.qweight, (unsigned)((size_t)(a.K >> 3) * a.N * 4));
        const int vw = live ? (((k0 >> 3) + kk) * a.N + col) * 4 : 0;
#pragma unroll
        for (int t = 0; t < NSTEP; ++t) wv[t] = buf_load128_stream(rw, vw, off + 16 * t * a.N);
    }

    // Rows >= M of the A operand hold a copy of row M-1: harmless, a row of A only reaches the same row of
    // the product, and rows >= M of the product are never stored.
    __device__ __forceinline__ void load_x(const half_t* row_chunk) {
#pragma unroll
        for (int t = 0; t < NSTEP; ++t) xv[t] = *reinterpret_cast<const uint4_t*>(row_chunk + 32 * t);
    }

    __device__ __forceinline__ void multiply(const GemvArgs& a, float4_t yacc[4], int c) const {
        // B operands of the two extra MFMAs: per-position offsets (1024 | 64) and all ones
        const half8_t offs = make_half8(0x64006400u, 0x54005400u, 0x64006400u, 0x54005400u);
        const half8_t ones = make_half8(0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u);
        // pass 1 (needs the activations only): A operands and the two weight-independent products
        half8_t av[NSTEP];
        float4_t acco_g[NG], accx_g[NG];
#pragma unroll
        for (int gi = 0; gi < NG; ++gi) {
            acco_g[gi] = float4_t{0.f, 0.f, 0.f, 0.f};
            accx_g[gi] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int tt = 0; tt < GS; ++tt) {
                const int t = gi * GS + tt;
                av[t] = make_half8(__builtin_amdgcn_perm(xv[t].z, xv[t].x, 0x05040100u),
                                   __builtin_amdgcn_perm(xv[t].z, xv[t].x, 0x07060302u),
                                   __builtin_amdgcn_perm(xv[t].w, xv[t].y, 0x05040100u),
                                   __builtin_amdgcn_perm(xv[t].w, xv[t].y, 0x07060302u));
                acco_g[gi] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[t], offs, acco_g[gi], 0, 0, 0);
                accx_g[gi] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[t], ones, accx_g[gi], 0, 0, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int gi = 0; gi < NG; ++gi) {
            float4_t acc[4];
            const float4_t acco = acco_g[gi], accx = accx_g[gi];
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int tt = 0; tt < GS; ++tt) {
                const int t = gi * GS + tt;
                const uint32_t w[4] = {wv[t].x, wv[t].y, wv[t].z, wv[t].w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t hi = w[j] >> 8;
                    const half8_t bv = make_half8((w[j] & 0x000F000Fu) | 0x64006400u, (w[j] & 0x00F000F0u) | 0x54005400u,
                                                  (hi & 0x000F000Fu) | 0x64006400u, (hi & 0x00F000F0u) | 0x54005400u);
                    acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[t], bv, acc[j], 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);      // consume the loads in the order they return
            }
            const half2_t s01 = as_half2(sv[gi].x), s23 = as_half2(sv[gi].y);
            const float sf[4] = {(float)s01[0], (float)s01[1], (float)s23[0], (float)s23[1]};
            if constexpr (V1) {
                // y += s * (sum x*(off+q) - sum x*off) - zero * sum x
                const half2_t z01 = as_half2(zh.x), z23 = as_half2(zh.y);
                const float zf[4] = {(float)z01[0], (float)z01[1], (float)z23[0], (float)z23[1]};
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (r < a.M) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) yacc[j][r] += sf[j] * (acc[j][r] - acco[r]) - zf[j] * accx[r];
                    }
                }
            } else {
                // group epilogue: y += s * ((sum x*(off+q) - sum x*off) - (z+1) * sum x)
                const uint32_t zw = zv[gi] >> ((c & 1) * 16);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (r < a.M) {                      // uniform: with M <= 3 the other accumulator rows are unused
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const float zf = (float)(((zw >> (4 * j)) & 0xFu) + 1u);
                            yacc[j][r] += sf[j] * ((acc[j][r] - acco[r]) - zf * accx[r]);
                        }
                    }
                }
            }
        }
    }
};

// `split` of `S`: which part of K this workgroup takes.
template <int NSTEP, int GSTEPS, bool V1>
__device__ __forceinline__ void gemv_seq_body(const GemvArgs& a, int n0, int split, int S) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nwaves = blockDim.x >> 6;
    const int kk = lane >> 4, c = lane & 15;
    const int k0 = (split * nwaves + wave) * (32 * NSTEP);

    float4_t yacc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) yacc[j] = float4_t{0.f, 0.f, 0.f, 0.f};

    if (k0 < a.K) {                               // wave-uniform; K % (32*NSTEP) == 0 (checked on the host)
        SeqChunk<NSTEP, GSTEPS, V1> ch;
        // activations first: they come from the caches and return early, so the operand shuffles and the two
        // weight-independent products run while the packed words are still on their way from HBM
        ch.load_x(a.x + (size_t)min(c, a.M - 1) * a.K + k0 + 8 * kk);
        ch.load_weights(a, k0, n0 + 4 * c, kk);
        // Keep the burst a burst: the scheduler must not sink loads below the arithmetic.
        __builtin_amdgcn_sched_barrier(0);
        ch.multiply(a, yacc, c);
    }
    gemv_finish(a, yacc, n0, wave, nwaves, kk, c, S);
}

// ------------------------------------------------------------------ launch plan
struct GemvPlan {
    int nstep, gsteps, waves, splits;
};

inline bool group_compatible(int gs32, int nstep, int* gsteps) {
    if (gs32 % nstep == 0) { *gsteps = 0; return true; }
    if (gs32 < nstep && nstep % gs32 == 0 && (gs32 == 1 || gs32 == 2 || gs32 == 4 || gs32 == 8)) { *gsteps = gs32; return true; }
    return false;
}

// Largest chunk (<= max_nstep steps) that divides K and is compatible with the grouping; 8 waves
// per workgroup reduce through LDS, the rest of K goes to gridDim.y (measured best on MI355X:
// ~700 workgroups of 512 threads for the LLaMA-7B MLP shapes).
inline GemvPlan plan_gemv(int K, int N, int groupsize, bool seq, int max_nstep) {
    const int steps = K / 32;
    const int gs32 = seq ? groupsize / 32 : 1;
    GemvPlan p{1, 0, 1, 1};
    for (int ns : {16, 8, 4, 2, 1}) {
        if (ns > max_nstep || steps % ns) continue;
        int gst = 0;
        if (seq && !group_compatible(gs32, ns, &gst)) continue;
        p.nstep = ns; p.gsteps = gst;
        break;
    }
    const int chunks = steps / p.nstep;
    const int strips = N / kColsPerWave;
    (void)strips;
    int waves = 8;
    const int max_waves = (!seq || p.nstep >= 16) ? 8 : 16;      // register budget of the kernels' launch bounds
    if (waves > chunks) waves = chunks;
    if (waves > max_waves) waves = max_waves;
    if (waves < 1) waves = 1;
    p.waves = waves;
    p.splits = (chunks + waves - 1) / waves;
    if (p.splits > 255) {                                        // 8-bit arrival counter
        p.waves = max_waves;
        p.splits = (chunks + max_waves - 1) / max_waves;
    }
    return p;
}

}  // namespace q4
