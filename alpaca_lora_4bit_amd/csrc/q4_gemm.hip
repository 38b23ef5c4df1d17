// Fused dequantize + fp16 MFMA GEMMs (MFMA-bound):
//   forward   y [M,N] = x  [M,K] @ W      (+ bias) (+ xa  [M,R] @ lora_bt [R,N])
//   backward  dx[M,K] = dy [M,N] @ W^T             (+ dyb [M,R] @ lora_a  [R,K])
// W is never materialised in HBM: each workgroup dequantizes the [64 x 128] slab of W its
// current step needs straight into LDS, with the reference's three fp16 roundings
// (src/alpaca_lora_4bit/quant_cuda/quant_cuda_kernel.cu:1146-1151), so the product equals
// torch.matmul(x, recons(W)) of matmul_utils_4bit.py:122-126 up to fp32 summation order.
//
// Tiling.  Workgroup = 256 threads = 4 wavefronts in a 2 x 2 arrangement over a 128 x 128
// output tile; each wavefront holds 2 x 2 accumulators of v_mfma_f32_32x32x16_f16 (64 fp32
// registers per lane).  The reduction runs in steps of 64.  Both LDS tiles are stored
// "row = output index, minor = reduction index" with 8 halves of padding per row (stride
// 144 B), which makes the 128-bit operand fetches of 16 consecutive lanes hit 64 distinct banks.
// Global loads of step t+1 are issued before the MFMAs of step t and land in registers.
//
// The LoRA term is one more reduction step whose A operand is the precomputed [M,R] rank-R
// activation and whose B operand is the fp16 adapter matrix: no second pass over the output.
#include "q4_common.hpp"
#include <type_traits>

namespace q4 {

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int LDS_STRIDE = BK + 8;   // halves

struct GemmArgs {
    const half_t* a;          // fwd: x [M,K]      bwd: dy [M,N]
    const uint32_t* qweight;  // [K/8, N]
    const uint32_t* qzeros;   // [G, N/8]
    const half_t* scales;     // [G, N]
    const int32_t* g_idx;     // [K] or null
    int groupsize;
    const half_t* bias;       // fwd only, [N] or null
    const half_t* la;         // fwd: xa [M,R]     bwd: dyb [M,R]   (or null)
    const half_t* lb;         // fwd: lora_bt [R,N] bwd: lora_a [R,K]
    int R;
    half_t* out;              // fwd: y [M,N]      bwd: dx [M,K]
    int M, K, N;
};

// ---- weight slab loaders: global -> registers -> (dequant) -> LDS ----------------------
// Forward: slab = 64 rows (k) x 128 columns (n); LDS row = column n, minor = k.
// A thread owns ONE column for the whole kernel and 4 packed words (32 rows) per step.
template <bool GIDX>
struct FwdSlab {
    uint32_t w[4];
    int col;        // 0..127 within the tile
    int wr0;        // first word-row within the slab (0 or 1), then +2 per word
    __device__ __forceinline__ void init(int t) { col = t & 127; wr0 = t >> 7; }
    __device__ __forceinline__ void load(const GemmArgs& a, int n0, int kred0) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            w[i] = a.qweight[(size_t)((kred0 >> 3) + wr0 + 2 * i) * a.N + n0 + col];
    }
    __device__ __forceinline__ void store(const GemmArgs& a, int n0, int kred0, half_t* sB) const {
        const int n = n0 + col;
        const int ncol8 = a.N >> 3;
        const int zsh = (n & 7) * 4;
        half2_t s2, zero2;
        if (!GIDX) {
            const int g = kred0 / a.groupsize;
            const half_t s = a.scales[(size_t)g * a.N + n];
            const uint32_t z = (a.qzeros[(size_t)g * ncol8 + (n >> 3)] >> zsh) & 0xFu;
            s2 = half2_t{s, s};
            zero2 = zero_term(s2, z, z);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int wr = wr0 + 2 * i;
            half2_t q2[4];
            unpack8_natural(w[i], q2);
            uint32_t o[4];
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                if (GIDX) {
                    const int k = kred0 + 8 * wr + 2 * p;
                    const int g0 = a.g_idx[k], g1 = a.g_idx[k + 1];
                    s2 = half2_t{a.scales[(size_t)g0 * a.N + n], a.scales[(size_t)g1 * a.N + n]};
                    zero2 = zero_term(s2, (a.qzeros[(size_t)g0 * ncol8 + (n >> 3)] >> zsh) & 0xFu,
                                      (a.qzeros[(size_t)g1 * ncol8 + (n >> 3)] >> zsh) & 0xFu);
                }
                o[p] = as_u32(dequant_pair(q2[p], s2, zero2));
            }
            *reinterpret_cast<uint4_t*>(sB + col * LDS_STRIDE + 8 * wr) = uint4_t{o[0], o[1], o[2], o[3]};
        }
    }
    // LoRA step: B operand = lora_bt [R, N]; LDS row = column n, minor = r (zero padded to 64).
    __device__ __forceinline__ void store_lora(const GemmArgs& a, int n0, half_t* sB, int t) const {
        for (int idx = t; idx < BN * BK; idx += 256) {
            const int r = idx >> 7, c = idx & 127;
            sB[c * LDS_STRIDE + r] = (r < a.R) ? a.lb[(size_t)r * a.N + n0 + c] : (half_t)0.f;
        }
    }
};

// Backward: output columns are rows k of W, the reduction runs over n.
// Slab = 128 rows (k) x 64 columns (n); LDS row = k, minor = n.
// A thread owns one word-row (8 output rows) and 4 adjacent columns per step (one 128-bit load).
template <bool GIDX>
struct BwdSlab {
    uint4_t w;
    int wr, n4;
    __device__ __forceinline__ void init(int t) { wr = t >> 4; n4 = t & 15; }
    __device__ __forceinline__ void load(const GemmArgs& a, int kout0, int nred0) {
        w = *reinterpret_cast<const uint4_t*>(a.qweight + (size_t)((kout0 >> 3) + wr) * a.N + nred0 + 4 * n4);
    }
    __device__ __forceinline__ void store(const GemmArgs& a, int kout0, int nred0, half_t* sB) const {
        const int n = nred0 + 4 * n4;
        const int ncol8 = a.N >> 3;
        const int zsh = (n & 7) * 4;    // 0 or 16
        const int kbase = kout0 + 8 * wr;
        const uint32_t wj[4] = {w.x, w.y, w.z, w.w};
        uint32_t lo[4], hi[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) { lo[j] = wj[j] & 0x0F0F0F0Fu; hi[j] = (wj[j] >> 4) & 0x0F0F0F0Fu; }
        half2_t s01, s23, z01, z23;
        auto fetch = [&](int g) {
            const uint2_t sv = *reinterpret_cast<const uint2_t*>(a.scales + (size_t)g * a.N + n);
            const uint32_t zw = a.qzeros[(size_t)g * ncol8 + (n >> 3)] >> zsh;
            s01 = as_half2(sv.x); s23 = as_half2(sv.y);
            z01 = zero_term(s01, zw & 0xFu, (zw >> 4) & 0xFu);
            z23 = zero_term(s23, (zw >> 8) & 0xFu, (zw >> 12) & 0xFu);
        };
        if (!GIDX) fetch(kbase / a.groupsize);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            if (GIDX) fetch(a.g_idx[kbase + e]);
            const int b = e >> 1;
            const uint32_t sel = 0x0c000c00u | ((4u + b) << 16) | (uint32_t)b;
            // (code of column j, code of column j+1) of row e
            const uint32_t c01 = (e & 1) ? __builtin_amdgcn_perm(hi[1], hi[0], sel) : __builtin_amdgcn_perm(lo[1], lo[0], sel);
            const uint32_t c23 = (e & 1) ? __builtin_amdgcn_perm(hi[3], hi[2], sel) : __builtin_amdgcn_perm(lo[3], lo[2], sel);
            const uint2_t o = {as_u32(dequant_pair(codes_to_half2(c01), s01, z01)),
                               as_u32(dequant_pair(codes_to_half2(c23), s23, z23))};
            *reinterpret_cast<uint2_t*>(sB + (8 * wr + e) * LDS_STRIDE + 4 * n4) = o;
        }
    }
    // LoRA step: B operand = lora_a [R, K]; LDS row = k, minor = r.
    __device__ __forceinline__ void store_lora(const GemmArgs& a, int kout0, half_t* sB, int t) const {
        for (int idx = t; idx < BN * BK; idx += 256) {
            const int r = idx >> 7, c = idx & 127;
            sB[c * LDS_STRIDE + r] = (r < a.R) ? a.lb[(size_t)r * a.K + kout0 + c] : (half_t)0.f;
        }
    }
};

// FWD: out[M, NOUT=N], reduction length RED=K.   BWD: out[M, NOUT=K], reduction length RED=N.
template <bool FWD, bool GIDX>
__global__ __launch_bounds__(256) void gemm_kernel(GemmArgs a) {
    __shared__ __attribute__((aligned(16))) half_t sA[BM * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) half_t sB[BN * LDS_STRIDE];

    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int NOUT = FWD ? a.N : a.K;
    const int RED = FWD ? a.K : a.N;
    const int m0 = blockIdx.y * BM;
    const int c0 = blockIdx.x * BN;          // first output column of the tile

    // activation tile: 128 rows x 64 reduction entries, 16 B per thread per pass, 4 passes
    const int arow = t >> 3, acol = (t & 7) * 8;
    uint4_t areg[4];
    auto load_a = [&](const half_t* base, int ld, int red0, int redlen) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int m = m0 + arow + 32 * i;
            areg[i] = uint4_t{0u, 0u, 0u, 0u};
            if (m < a.M && red0 + acol < redlen)
                areg[i] = *reinterpret_cast<const uint4_t*>(base + (size_t)m * ld + red0 + acol);
        }
    };
    auto store_a = [&]() {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            *reinterpret_cast<uint4_t*>(sA + (arow + 32 * i) * LDS_STRIDE + acol) = areg[i];
    };

    typename std::conditional<FWD, FwdSlab<GIDX>, BwdSlab<GIDX>>::type slab;
    slab.init(t);

    float16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    auto mma_tile = [&](int ksteps) {
        const int lr = lane & 31, lk = (lane >> 5) * 8;
        for (int ks = 0; ks < ksteps; ++ks) {
            half8_t af[2], bf[2];
#pragma unroll
            for (int i = 0; i < 2; ++i)
                af[i] = *reinterpret_cast<const half8_t*>(sA + (wm * 64 + 32 * i + lr) * LDS_STRIDE + 16 * ks + lk);
#pragma unroll
            for (int j = 0; j < 2; ++j)
                bf[j] = *reinterpret_cast<const half8_t*>(sB + (wn * 64 + 32 * j + lr) * LDS_STRIDE + 16 * ks + lk);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
    };

    const int nsteps = RED / BK;
    load_a(a.a, RED, 0, RED);
    slab.load(a, c0, 0);
    for (int s = 0; s < nsteps; ++s) {
        store_a();
        slab.store(a, c0, s * BK, sB);
        __syncthreads();
        if (s + 1 < nsteps) {
            load_a(a.a, RED, (s + 1) * BK, RED);
            slab.load(a, c0, (s + 1) * BK);
        }
        mma_tile(BK / 16);
        __syncthreads();
    }
    if (a.R > 0) {
        load_a(a.la, a.R, 0, a.R);
        store_a();
        slab.store_lora(a, c0, sB, t);
        __syncthreads();
        mma_tile((a.R + 15) / 16);
    }

    // epilogue: acc[i][j][r] is row 8*(r/4) + 4*(lane/32) + r%4, column lane%32 of its 32x32 tile
    const int lc = lane & 31, lrow = (lane >> 5) * 4;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int col = c0 + wn * 64 + 32 * j + lc;
        const float bv = (FWD && a.bias) ? (float)a.bias[col] : 0.f;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm * 64 + 32 * i + 8 * (r >> 2) + lrow + (r & 3);
                if (m < a.M) a.out[(size_t)m * NOUT + col] = (half_t)(acc[i][j][r] + bv);
            }
    }
}

}  // namespace q4

extern "C" int q4_launch_gemm(int fwd, const void* act, const int32_t* qweight, const int32_t* qzeros,
                              const void* scales, const int32_t* g_idx, int groupsize, const void* bias,
                              const void* la, const void* lb, int R, void* out, int M, int K, int N,
                              hipStream_t stream) {
    using namespace q4;
    GemmArgs a;
    a.a = reinterpret_cast<const half_t*>(act);
    a.qweight = reinterpret_cast<const uint32_t*>(qweight);
    a.qzeros = reinterpret_cast<const uint32_t*>(qzeros);
    a.scales = reinterpret_cast<const half_t*>(scales);
    a.g_idx = g_idx;
    a.groupsize = groupsize;
    a.bias = reinterpret_cast<const half_t*>(bias);
    a.la = reinterpret_cast<const half_t*>(la);
    a.lb = reinterpret_cast<const half_t*>(lb);
    a.R = (la && lb) ? R : 0;
    a.out = reinterpret_cast<half_t*>(out);
    a.M = M; a.K = K; a.N = N;
    const int nout = fwd ? N : K;
    const dim3 grid(nout / BN, (M + BM - 1) / BM);
    const dim3 block(256);
    const bool gidx = g_idx != nullptr;
    if (fwd) {
        if (gidx) hipLaunchKernelGGL((gemm_kernel<true, true>), grid, block, 0, stream, a);
        else hipLaunchKernelGGL((gemm_kernel<true, false>), grid, block, 0, stream, a);
    } else {
        if (gidx) hipLaunchKernelGGL((gemm_kernel<false, true>), grid, block, 0, stream, a);
        else hipLaunchKernelGGL((gemm_kernel<false, false>), grid, block, 0, stream, a);
    }
    return hipGetLastError() == hipSuccess ? 0 : -4;
}
