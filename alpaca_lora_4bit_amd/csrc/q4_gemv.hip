// Weight-streaming products for few activation rows:  y[M,N] = x[M,K] @ W   (HBM-bound).
//   gemv_seq_kernel       1 <= M <= 16, sequential groups (also the v1 layout: one scale / zero per column)
//   gemv_seq_perm_kernel  1 <= M <= 4, act-order layer with rows sorted by group: gathers x through the permutation
//   gemv_gidx_kernel      1 <= M <= 16, act-order with per-row groups read through g_idx
//   skinny_seq_kernel     17 <= M <= 64, sequential groups (fp32 partial rows + ordered reduction)
//   skinny_dx_kernel      17 <= M <= 48, the transposed product dy @ W^T (grad-input), sequential groups
//
// Work split.  A workgroup owns a strip of 64 columns; its W wavefronts (W = blockDim.x / 64)
// take consecutive chunks of 32*NSTEP rows, and gridDim.y workgroups share one strip when K is
// longer than W chunks.  Lane l of a wavefront (kk = l / 16, c = l % 16) reads, per step of 32
// rows, ONE 128-bit vector qweight[row/8 + kk, n0 + 4c .. 4c+3]: four packed words = 8
// consecutive rows of four adjacent columns.  A packed word is exactly the 8-deep k-slice that
// lane l feeds to v_mfma_f32_16x16x32_f16 as its B operand, so the four words go to four MFMAs
// whose column index i stands for column n0 + 4i + j (j = 0..3).  The A operand is x (row
// m = l % 16, the same 8 k values; rows >= M repeat row M-1), so all M <= 16 activation rows ride
// along and the weights are read from HBM once.  Every load of a chunk is issued before the
// first is consumed, in straight-line code: with ~90 KB of weights per CU the kernel is one
// burst of loads followed by a short arithmetic tail.
//
// Sequential groups (no act-order).  The B operand holds the raw codes as fp16 (1024 + q for the
// nibbles in bits 0-3 of a half, 64 + q for those in bits 4-7) and two more MFMAs with constant B
// operands yield O = sum_k x*offset and X = sum_k x over the same rows, so per group only
//   y += s * ((acc - O) - (z + 1) * X)   is evaluated (fp32) instead of one multiply-subtract per
// weight.  Mathematically equal to sum_k x*(s*q - s*(z+1))
// (src/alpaca_lora_4bit/quant_cuda/quant_cuda_kernel.cu:1026-1037); not bit-identical to it,
// nor is the reference to itself (fp16 partial sums and atomicAdd order, :1037,1040).
//
// Act-order.  Rows of one word can belong to 8 different groups, so the B operand is built
// from explicitly dequantized weights with (scale, zero) gathered through g_idx per row
// (the convention of VecQuant4MatMulKernel, quant_cuda_kernel.cu:513-520).
//
// Reduction over K.  Inside a workgroup: through LDS.  Across the gridDim.y workgroups of a
// strip: ONE 64-bit integer atomic per output element.  The fp32 partial is converted to
// fixed point (24 fractional bits, biased to stay non-negative) in the low 56 bits, the top 8
// bits count arrivals; the workgroup whose atomic returns count == gridDim.y - 1 holds the
// complete sum, writes y and stores 0 back.  Integer addition is associative, so the result
// is independent of arrival order (bit-reproducible), and the whole exchange costs a single
// memory round trip, with no fences and no spinning.
#include "q4_common.hpp"
#include "q4_gptq.h"
#include <stdlib.h>
#include <type_traits>

#include "q4_gemv_core.hpp"

namespace q4 {

template <int NSTEP, int GSTEPS, bool V1 = false>
__global__ __launch_bounds__(NSTEP >= 16 ? 512 : 1024) void gemv_seq_kernel(GemvArgs a) {
    gemv_seq_body<NSTEP, GSTEPS, V1>(a, blockIdx.x * kColsPerWave, blockIdx.y, gridDim.y);
}

// Up to kMaxGroup layers with the same K, group size and row count M in ONE grid (q|k|v or gate|up of a decoder
// block, read in place from their own tensors): blockIdx.x walks the strips of layer 0, then of layer 1, ...
// A launch costs about 3 us of fixed time (dispatch, ramp, the reduction round trip) on top of the streaming
// time of its bytes, so two or three layers in one launch run close to the time of the largest alone.
constexpr int kMaxGroup = 4;
struct GemvGroupArgs {
    GemvArgs layer[kMaxGroup];
    int strip_end[kMaxGroup];                     // running total of 64-column strips; unused entries = INT_MAX
};

template <int NSTEP, int GSTEPS>
__global__ __launch_bounds__(1024) void gemv_seq_group_kernel(GemvGroupArgs g) {
    const int bx = blockIdx.x;
    const int li = (bx >= g.strip_end[0]) + (bx >= g.strip_end[1]) + (bx >= g.strip_end[2]);      // uniform
    const int first = li == 0 ? 0 : g.strip_end[li - 1];
    gemv_seq_body<NSTEP, GSTEPS, false>(g.layer[li], (bx - first) * kColsPerWave, blockIdx.y, gridDim.y);
}

// The same for an act-order layer whose packed rows were sorted by group (q4_permute_rows): row p of the
// sorted matrix is row perm[p] of the original, so the product needs x[:, perm[p]].  Gathering from global
// memory would cost one scattered request per element in every strip's workgroups; instead the workgroup copies
// the whole activation rows into LDS with coalesced loads (M*K*2 bytes, small for M <= 4), gathers the
// entries of its K range from there into the operand tile and continues as the kernel above.  The
// permutation entries are requested first and the weights right after, so everything is in flight together.
// LDS: reduction buffer [nwaves][M][64] fp32, operand tile [M][span] fp16, activation rows [M][K] fp16.
template <int NSTEP, int GSTEPS>
__global__ __launch_bounds__(1024) void gemv_seq_perm_kernel(GemvArgs a) {
    extern __shared__ float red[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nwaves = blockDim.x >> 6;
    const int kk = lane >> 4, c = lane & 15;
    const int n0 = blockIdx.x * kColsPerWave;
    const int span = nwaves * 32 * NSTEP;          // reduction rows of this workgroup
    const int kbase = blockIdx.y * span;
    const int k0 = kbase + wave * (32 * NSTEP);
    const bool active = k0 < a.K;                  // wave-uniform
    half_t* xs = reinterpret_cast<half_t*>(red + ((nwaves * a.M) << 6));     // [M][span]
    half_t* xfull = xs + a.M * span;                                          // [M][K]

    float4_t yacc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) yacc[j] = float4_t{0.f, 0.f, 0.f, 0.f};

    // No branch sits between the loads below (out-of-range pieces come back as zeros), so the compiler's wait
    // before the first use of the early ones does not include the weights.
    constexpr int PT = 2;                          // reduction rows per thread: span <= 2 * blockDim.x
    constexpr int XT = 8;                          // 16-byte pieces of x per thread: M*K*2 <= 64 KB with 512 threads
    const rsrc_t rp = make_rsrc(a.perm, (unsigned)a.K * 4u);
    const rsrc_t rx = make_rsrc(a.x, (unsigned)(a.M * a.K) * 2u);
    int src[PT];
#pragma unroll
    for (int u = 0; u < PT; ++u) src[u] = (int)buf_load32(rp, (kbase + (int)threadIdx.x + u * (int)blockDim.x) * 4, 0);
    uint4_t xc[XT];
#pragma unroll
    for (int u = 0; u < XT; ++u) xc[u] = buf_load128(rx, ((int)threadIdx.x + u * (int)blockDim.x) * 16, 0);
    SeqChunk<NSTEP, GSTEPS> ch;
    ch.load_weights_branch_free(a, k0, n0 + 4 * c, kk, active);
    __builtin_amdgcn_sched_barrier(0);
    const int n16 = (a.M * a.K) >> 3;              // K % 32 == 0
#pragma unroll
    for (int u = 0; u < XT; ++u) {
        const int i = threadIdx.x + u * blockDim.x;
        if (i < n16) reinterpret_cast<uint4_t*>(xfull)[i] = xc[u];
    }
    __syncthreads();
    {
        half_t got[PT][4];                         // all LDS reads first, then the writes: one LDS latency, not 2*M
#pragma unroll
        for (int u = 0; u < PT; ++u)
#pragma unroll
            for (int m = 0; m < 4; ++m) got[u][m] = xfull[min(m, a.M - 1) * a.K + src[u]];
#pragma unroll
        for (int u = 0; u < PT; ++u) {
            const int i = threadIdx.x + u * blockDim.x;
            if (i < span && kbase + i < a.K) {
#pragma unroll
                for (int m = 0; m < 4; ++m)
                    if (m < a.M) xs[m * span + i] = got[u][m];
            }
        }
    }
    __syncthreads();
    if (active) {
        ch.load_x(xs + min(c, a.M - 1) * span + (k0 - kbase) + 8 * kk);
        __builtin_amdgcn_sched_barrier(0);
        ch.multiply(a, yacc, c);
    }
    gemv_finish(a, yacc, n0, wave, nwaves, kk, c, gridDim.y);
}

// ------------------------------------------------------------------ 17 <= M <= 64 (sequential groups)
// The same streaming scheme for RB blocks of 16 activation rows.  A wavefront owns one chunk of 128
// reduction rows: it loads that chunk of every activation row once, keeps it as MFMA A operands in
// registers (together with the two offset products, which do not depend on the weights) and walks over
// `strips_per_wg` neighbouring 64-column strips, prefetching the packed weights of the next strip while it
// multiplies the current one - so the activations are read once per strips_per_wg strips, not once per
// strip.  The B operands are rebuilt from the words (five ALU ops each) once per strip and used for every
// row block.  The eight wavefronts of a workgroup (eight chunks) are summed through LDS; with M rows per
// strip the cross-workgroup sum would need M*64 atomics per workgroup, so the workgroups of a strip
// leave fp32 partial rows in a scratch buffer [gridDim.y][M][N] instead and a second kernel adds them in
// order (bit-reproducible); the bias rides with split 0.
// Chunks of 128 rows inside one quantization group only (groupsize % 128 == 0).  No branches around the
// loads: a wavefront past the end of K, and the prefetch after the last strip, fetch from an offset
// beyond every buffer, which returns zeros without traffic.
struct SkinnyArgs {
    const half_t* x;
    const uint32_t* qweight;
    const uint32_t* qzeros;
    const half_t* scales;
    const half_t* bias;       // [N] or null
    int groupsize;
    half_t* y;                // written directly when gridDim.y == 1
    float* part;              // [gridDim.y][M][N]
    int M, K, N, G;           // G: rows of scales / qzeros (ceil(K / groupsize): the last group may be partial)
    int strips_per_wg;
};

template <int RB>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(RB <= 2 ? 4 : 2)))
void skinny_seq_kernel(SkinnyArgs a) {
    constexpr int NSTEP = 4, NW = 8;
    constexpr int kFar = 0x70000000;
    // [row block][wavefront][row][column of the strip]; before the first strip, the activation tiles
    __shared__ __attribute__((aligned(16))) float red[RB][NW][16 * 64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kk = lane >> 4, c = lane & 15;
    const int strip0 = blockIdx.x * a.strips_per_wg;
    const int nl = min(a.strips_per_wg, (a.N >> 6) - strip0);
    const int k0 = (blockIdx.y * NW + wave) * (32 * NSTEP);
    const int dead = k0 < a.K ? 0 : kFar;          // wave-uniform
    const int G = a.G, g = dead ? 0 : k0 / a.groupsize;
    const int S = gridDim.y;

    const rsrc_t rw = make_rsrc(a.qweight, (unsigned)((size_t)(a.K >> 3) * a.N * 4));
    const rsrc_t rs = make_rsrc(a.scales, (unsigned)((size_t)G * a.N * 2));
    const rsrc_t rz = make_rsrc(a.qzeros, (unsigned)((size_t)G * (a.N >> 3) * 4));
    const rsrc_t rx = make_rsrc(a.x, (unsigned)((size_t)a.M * a.K * 2));
    // the bias rides with split 0; an empty buffer reads as zeros
    const rsrc_t rb_bias = make_rsrc(a.bias, a.bias && blockIdx.y == 0 ? (unsigned)a.N * 2 : 0u);
    const int vw = dead ? 0 : (((k0 >> 3) + kk) * a.N + 4 * c) * 4;
    const int vs = (g * a.N + 4 * c) * 2;
    const int vz = (g * (a.N >> 3) + (c >> 1)) * 4;
    const int wstep = 16 * a.N;                    // bytes between the words of two steps (4 packed rows)

    uint4_t wv[NSTEP];
    uint2_t sv;
    uint32_t zv;
    // Activations: a lane of the MFMA A operand wants 16 bytes of row c, so a direct load would touch 16
    // rows (16 cache lines) per quarter wavefront and the vector cache would spend its time on tag lookups.
    // Load row-contiguous instead (a quarter wavefront = 256 contiguous bytes of one row) and turn the tile
    // through this wavefront's own 4 KB of LDS per row block: 16 rows x 16 units of 16 bytes, unit q of
    // row r stored at q ^ r, which keeps both the row-wise writes and the column-wise reads conflict-free.
    half8_t av[RB][NSTEP];
    {
        uint4_t xv[RB][NSTEP];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int i = 0; i < NSTEP; ++i) {
                // rows >= M hold a copy of row M-1: they only reach rows of the product that are never stored
                const int vx = (min(16 * rb + 4 * i + kk, a.M - 1) * a.K + 8 * c) * 2;
                xv[rb][i] = buf_load128(rx, vx, dead + k0 * 2);
            }
        // the weights of the first strip right behind the activations: those come from the caches and return
        // first (loads return in issue order), so the turn through LDS and the offset products below run while
        // the packed words are still on their way from HBM
        sv = buf_load64(rs, vs, dead + strip0 * 128);
        zv = buf_load32(rz, vz, dead + strip0 * 32);
#pragma unroll
        for (int t = 0; t < NSTEP; ++t) wv[t] = buf_load128(rw, vw, dead + strip0 * 256 + t * wstep);
        __builtin_amdgcn_sched_barrier(0);        // one burst of loads, nothing sunk below the arithmetic
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            uint4_t* stage = reinterpret_cast<uint4_t*>(&red[rb][wave][0]);
#pragma unroll
            for (int i = 0; i < NSTEP; ++i) stage[(4 * i + kk) * 16 + (c ^ (4 * i + kk))] = xv[rb][i];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // A operands in the order the nibble split below produces: (e0,e4)(e1,e5)(e2,e6)(e3,e7)
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            const uint4_t* stage = reinterpret_cast<const uint4_t*>(&red[rb][wave][0]);
#pragma unroll
            for (int t = 0; t < NSTEP; ++t) {
                const uint4_t u = stage[c * 16 + ((4 * t + kk) ^ c)];
                av[rb][t] = make_half8(__builtin_amdgcn_perm(u.z, u.x, 0x05040100u), __builtin_amdgcn_perm(u.z, u.x, 0x07060302u),
                                       __builtin_amdgcn_perm(u.w, u.y, 0x05040100u), __builtin_amdgcn_perm(u.w, u.y, 0x07060302u));
            }
        }
    }
    // sum x*offset and sum x of the chunk: the same for every strip
    const half8_t offs = make_half8(0x64006400u, 0x54005400u, 0x64006400u, 0x54005400u);
    const half8_t ones = make_half8(0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u);
    float4_t acco[RB], accx[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        acco[rb] = float4_t{0.f, 0.f, 0.f, 0.f};
        accx[rb] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < NSTEP; ++t) {
            acco[rb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[rb][t], offs, acco[rb], 0, 0, 0);
            accx[rb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[rb][t], ones, accx[rb], 0, 0, 0);
        }
    }

    for (int l = 0; l < nl; ++l) {
        const int n0 = (strip0 + l) << 6;
        const int next = (dead || l + 1 >= nl) ? kFar : 0;    // uniform
        // bias of the two columns this thread finishes, ahead of the prefetch so that waiting for it
        // leaves the prefetch in flight
        const uint32_t bias2 = buf_load32(rb_bias, (2 * (int)threadIdx.x & 63) * 2, n0 * 2);
        uint4_t wn[NSTEP];
        const uint2_t sn = buf_load64(rs, vs, next + (strip0 + l + 1) * 128);
        const uint32_t zn = buf_load32(rz, vz, next + (strip0 + l + 1) * 32);
#pragma unroll
        for (int t = 0; t < NSTEP; ++t) wn[t] = buf_load128(rw, vw, next + (strip0 + l + 1) * 256 + t * wstep);
        __builtin_amdgcn_sched_barrier(0);

        float4_t acc[RB][4];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[rb][j] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < NSTEP; ++t) {
            const uint32_t w[4] = {wv[t].x, wv[t].y, wv[t].z, wv[t].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                // a code in mantissa bits 0..3 of fp16 1024.0 reads 1024 + q, in bits 4..7 of fp16 64.0 it reads 64 + q
                const uint32_t hi = w[j] >> 8;
                const half8_t bv = make_half8((w[j] & 0x000F000Fu) | 0x64006400u, (w[j] & 0x00F000F0u) | 0x54005400u,
                                              (hi & 0x000F000Fu) | 0x64006400u, (hi & 0x00F000F0u) | 0x54005400u);
#pragma unroll
                for (int rb = 0; rb < RB; ++rb)
                    acc[rb][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[rb][t], bv, acc[rb][j], 0, 0, 0);
            }
        }
        const uint32_t zw = zv >> ((c & 1) * 16);
        const half2_t s01 = as_half2(sv.x), s23 = as_half2(sv.y);
        const float sf[4] = {(float)s01[0], (float)s01[1], (float)s23[0], (float)s23[1]};
        // y = s * ((sum x*(off+q) - sum x*off) - (z+1) * sum x); row 4*kk + r of the block, columns 4c .. 4c+3
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float4_t v;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float zf = (float)(((zw >> (4 * j)) & 0xFu) + 1u);
                    v[j] = sf[j] * ((acc[rb][j][r] - acco[rb][r]) - zf * accx[rb][r]);
                }
                *reinterpret_cast<float4_t*>(&red[rb][wave][((4 * kk + r) << 6) + 4 * c]) = v;
            }
        __syncthreads();
        // sum over the wavefronts: thread t finishes row t/32 of every block, columns 2*(t%32) and the next
        {
            const int e = 2 * threadIdx.x;
            const int row = e >> 6, cc = n0 + (e & 63);
            const half2_t b2 = as_half2(bias2);
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                float v0 = 0.f, v1 = 0.f;
#pragma unroll
                for (int w = 0; w < NW; ++w) {
                    const float* rp = &red[rb][w][e];
                    v0 += rp[0];
                    v1 += rp[1];
                }
                const int m = 16 * rb + row;
                if (m < a.M) {
                    v0 += (float)b2[0];
                    v1 += (float)b2[1];
                    if (S == 1) {
                        const half2_t h = {(half_t)v0, (half_t)v1};
                        *reinterpret_cast<half2_t*>(a.y + (size_t)m * a.N + cc) = h;
                    } else {
                        float* pp = a.part + ((size_t)blockIdx.y * a.M + m) * a.N + cc;
                        pp[0] = v0;
                        pp[1] = v1;
                    }
                }
            }
        }
        __syncthreads();                           // red is rewritten for the next strip
#pragma unroll
        for (int t = 0; t < NSTEP; ++t) wv[t] = wn[t];
        sv = sn;
        zv = zn;
    }
}

// ------------------------------------------------------------------ forward, some hundred rows (sequential groups)
// Between the streaming kernel above and the tiled MFMA kernel lies a range of rows where an output has too few
// 256-row tiles to fill the CUs without splitting the reduction (partial tiles, a second kernel) and the kernel
// above pays its two barriers and an LDS sum per strip.  Here a workgroup owns one 64-column strip of 16*RB rows
// for the WHOLE reduction: wavefront w walks the chunks w, w + 8, ... of 128 reduction rows with its accumulators
// in registers, the next chunk's words, scales and activations in flight while it multiplies the current one, and
// the eight wavefronts are summed through LDS once, at the end, into fp16 outputs: one launch, no workspace.
// The B operand holds the dequantized weights rn16(rn16(s*q) - rn16(s*(z+1))) (the values of the dense kernel,
// quant_cuda_kernel.cu:1148-1152): with one scale per column of a chunk the product of code and scale is one
// packed fused multiply-add on (1024 + q) or (64 + q) (1024*s and 64*s are exact), the zero term one subtraction.
template <int RB>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2)))
void stream_fwd_kernel(SkinnyArgs a) {
    constexpr int NSTEP = 4, NW = 8;
    constexpr int kFar = 0x70000000;
    // [row block][wavefront][row][column of the strip]; inside the loop, the activation tiles being turned
    __shared__ __attribute__((aligned(16))) float red[RB][NW][16 * 64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kk = lane >> 4, c = lane & 15;
    const int n0 = blockIdx.x << 6;
    const int row0 = blockIdx.z * (16 * RB);
    const int nchunks = a.K >> 7;

    const rsrc_t rw = make_rsrc(a.qweight, (unsigned)((size_t)(a.K >> 3) * a.N * 4));
    const rsrc_t rs = make_rsrc(a.scales, (unsigned)((size_t)a.G * a.N * 2));
    const rsrc_t rz = make_rsrc(a.qzeros, (unsigned)((size_t)a.G * (a.N >> 3) * 4));
    const rsrc_t rx = make_rsrc(a.x, (unsigned)((size_t)a.M * a.K * 2));
    const int vw = (kk * a.N + n0 + 4 * c) * 4;
    const int vs = (n0 + 4 * c) * 2;
    const int vz = ((n0 >> 3) + (c >> 1)) * 4;
    const int wstep = 16 * a.N;                    // bytes between the words of two steps (4 packed rows)
    // Activations: a lane of the MFMA A operand wants 16 bytes of row c, so direct loads would touch 16 rows (16
    // cache lines) per quarter wavefront.  They are loaded row-contiguous instead (a quarter wavefront = 256
    // contiguous bytes of one row), straight into this wavefront's own 4 KB of LDS per row block (no registers in
    // between: the next chunk's tile travels while this chunk is multiplied), and read back column-wise.  Lane
    // (kk, c) of load i lands at unit c of row 4i + kk and fetches unit c ^ (4i + kk) of that row, so unit q of row
    // r sits at q ^ r: the column-wise reads are conflict-free.  Rows beyond M lie beyond the buffer: zeros.
    int vx[NSTEP];
#pragma unroll
    for (int i = 0; i < NSTEP; ++i) vx[i] = (kk * a.K + 8 * (c ^ (4 * i + kk))) * 2;
    typedef __attribute__((address_space(3))) void lds_void;

    uint4_t w0[NSTEP], w1[NSTEP];
    uint2_t sv;
    uint32_t zv;
    // everything chunk `ch` of this wavefront needs; past the end of the reduction: zeros, without traffic
    auto fetch = [&](int ch) {
        const int off = ch < nchunks ? 0 : kFar;
        const int k0 = ch << 7, g = k0 / a.groupsize;
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int i = 0; i < NSTEP; ++i)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_void*)(&red[rb][wave][256 * i]), 16, vx[i],
                                                         off + ((row0 + 16 * rb + 4 * i) * a.K + k0) * 2, 0, 0);
        sv = buf_load64(rs, vs, off + g * a.N * 2);
        zv = buf_load32(rz, vz, off + g * (a.N >> 3) * 4);
#pragma unroll
        for (int t = 0; t < NSTEP; ++t) w1[t] = buf_load128_stream(rw, vw, off + (ch << 4) * a.N * 4 + t * wstep);
    };
    fetch(wave);
    // mask (scalar register) and magic number (vector register) as opaque values: with two literals the compiler
    // emits an AND and an OR, with register operands the single three-operand and-or instruction
    uint32_t m_lo = 0x000F000Fu, m_hi = 0x00F000F0u, g_lo = 0x64006400u, g_hi = 0x54005400u;
    asm volatile("" : "+s"(m_lo), "+s"(m_hi));
    asm volatile("" : "+v"(g_lo), "+v"(g_hi));

    float4_t acc[RB][4];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[rb][j] = float4_t{0.f, 0.f, 0.f, 0.f};

    for (int ch = wave; ch < nchunks; ch += NW) {
        // the loads of this chunk have landed (vmcnt 0): the tile in LDS, words, scales and zeros in registers
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // A operands in the order the nibble split below produces: (e0,e4)(e1,e5)(e2,e6)(e3,e7)
        half8_t av[RB][NSTEP];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            const uint4_t* stage = reinterpret_cast<const uint4_t*>(&red[rb][wave][0]);
#pragma unroll
            for (int t = 0; t < NSTEP; ++t) {
                const uint4_t u = stage[c * 16 + ((4 * t + kk) ^ c)];
                av[rb][t] = make_half8(__builtin_amdgcn_perm(u.z, u.x, 0x05040100u), __builtin_amdgcn_perm(u.z, u.x, 0x07060302u),
                                       __builtin_amdgcn_perm(u.w, u.y, 0x05040100u), __builtin_amdgcn_perm(u.w, u.y, 0x07060302u));
            }
        }
        // scale and zero term of the four columns of this lane (one group per chunk)
        const uint32_t zw = zv >> ((c & 1) * 16);
        const uint32_t sraw[4] = {sv.x & 0xFFFFu, sv.x >> 16, sv.y & 0xFFFFu, sv.y >> 16};
        half2_t s2[4], s1024[4], s64[4], zero2[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const half2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f}, k64 = {(half_t)64.0f, (half_t)64.0f};
            s2[j] = as_half2(sraw[j] | (sraw[j] << 16));
            s1024[j] = s2[j] * k1024;
            s64[j] = s2[j] * k64;
            const uint32_t z = (zw >> (4 * j)) & 0xFu;
            zero2[j] = zero_term(s2[j], z, z);
        }
#pragma unroll
        for (int t = 0; t < NSTEP; ++t) w0[t] = w1[t];
        // the tile has been read (lgkmcnt 0): the next chunk of this wavefront may overwrite it
        __builtin_amdgcn_s_waitcnt(0xC07F);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_sched_barrier(0);
        fetch(ch + NW);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < NSTEP; ++t) {
            const uint32_t w[4] = {w0[t].x, w0[t].y, w0[t].z, w0[t].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                // a code in mantissa bits 0..3 of fp16 1024.0 reads 1024 + q, in bits 4..7 of fp16 64.0 it reads 64 + q
                const uint32_t hi = w[j] >> 8;
                const half2_t b0 = __builtin_elementwise_fma(as_half2((w[j] & m_lo) | g_lo), s2[j], -s1024[j]) - zero2[j];
                const half2_t b1 = __builtin_elementwise_fma(as_half2((w[j] & m_hi) | g_hi), s2[j], -s64[j]) - zero2[j];
                const half2_t b2 = __builtin_elementwise_fma(as_half2((hi & m_lo) | g_lo), s2[j], -s1024[j]) - zero2[j];
                const half2_t b3 = __builtin_elementwise_fma(as_half2((hi & m_hi) | g_hi), s2[j], -s64[j]) - zero2[j];
                const half8_t bv = make_half8(as_u32(b0), as_u32(b1), as_u32(b2), as_u32(b3));
#pragma unroll
                for (int rb = 0; rb < RB; ++rb)
                    acc[rb][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[rb][t], bv, acc[rb][j], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);     // B operands are built step by step, not all sixteen ahead
        }
    }
    // the prefetch past the last chunk of this wavefront wrote zeros into the tile: landed before the sum reuses it
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // sum over the wavefronts; row 4*kk + r of the block, columns 4c .. 4c+3
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int r = 0; r < 4; ++r)
            *reinterpret_cast<float4_t*>(&red[rb][wave][((4 * kk + r) << 6) + 4 * c]) =
                float4_t{acc[rb][0][r], acc[rb][1][r], acc[rb][2][r], acc[rb][3][r]};
    __syncthreads();
    {
        // thread t finishes row t/32 of every block, columns 2*(t%32) and the next
        const int e = 2 * threadIdx.x;
        const int row = e >> 6, cc = n0 + (e & 63);
        half2_t b2 = {(half_t)0.f, (half_t)0.f};
        if (a.bias) b2 = *reinterpret_cast<const half2_t*>(a.bias + cc);
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            float v0 = 0.f, v1 = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                const float* rp = &red[rb][w][e];
                v0 += rp[0];
                v1 += rp[1];
            }
            const int m = row0 + 16 * rb + row;
            if (m < a.M) {
                const half2_t h = {(half_t)(v0 + (float)b2[0]), (half_t)(v1 + (float)b2[1])};
                *reinterpret_cast<half2_t*>(a.y + (size_t)m * a.N + cc) = h;
            }
        }
    }
}

// ------------------------------------------------------------------ grad-input, 17 <= M <= 48 (sequential groups)
// dx[M, K] = dy[M, N] @ W^T with the same streaming scheme: the reduction runs over the columns n of W, the outputs
// are its rows k.  A packed word holds 8 consecutive rows k of one column n, so the 8 words of columns n .. n+7
// (two 128-bit loads of lane (i = l % 16, kk = l / 16): word-row k8 + i, columns n0 + 32*t + 8*kk .. + 7) hold an
// 8 x 8 block of codes, and nibble j of those 8 words is exactly the 8-deep slice of the reduction that lane l
// feeds to MFMA j as B operand for output row 8*(k8 + i) + j: eight MFMAs per step of 32 columns produce 16
// word-rows = 128 outputs, one quantization group when groupsize % 128 == 0.  Within a group the scale and the zero
// depend on n only, so they move to the A side:
//   dx[m, k] = sum_n (dy[m, n] * s[g, n]) * (1024 + q[k, n])  -  sum_n (dy[m, n] * s[g, n]) * (1025 + z[g, n])
// (codes enter as fp16 1024 + q by OR-ing them into the mantissa; the second sum is one more MFMA per step whose
// B operand is the same for all columns).  A wavefront owns one chunk of 128 columns n: it keeps that chunk of
// all dy rows as A operands in registers and walks over `strips_per_wg` neighbouring output blocks of 128 rows k,
// the words of the next two steps in flight while it multiplies.  The eight wavefronts of a workgroup (eight
// chunks) are summed through LDS, 64 outputs at a time; the gridDim.y workgroups of a block leave fp32 partial rows
// [gridDim.y][M][K] that gemm_splitk_reduce_kernel adds in order (bit-reproducible).
// Mathematically sum_n dy * W[k, n] (src/alpaca_lora_4bit/autograd_4bit.py:45-54 through
// matmul_utils_4bit.py:125-126); the scale is applied to dy before the product instead of to the weight, within
// the tolerance of the path.
template <int I, int N, typename F>
__device__ __forceinline__ void static_for_dx(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for_dx<I + 1, N>(f);
    }
}

struct SkinnyDxArgs {
    const half_t* dy;
    const uint32_t* qweight;
    const uint32_t* qzeros;
    const half_t* scales;
    int groupsize;
    half_t* dx;               // written directly when gridDim.y == 1
    float* part;              // [gridDim.y][M][K]
    int M, K, N, G;
    int strips_per_wg;
};

template <int RB, int SS>      // SS: steps of 32 columns per pipeline stage (2; 1 where registers are short)
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2)))
void skinny_dx_kernel(SkinnyDxArgs a) {
    constexpr int NSTEP = 4, NW = 8, NH = NSTEP / SS;
    constexpr int kFar = 0x70000000;
    __shared__ __attribute__((aligned(16))) float red[RB][NW][16 * 64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kk = lane >> 4, c = lane & 15;
    const int nblocks = a.K >> 7;
    const int strip0 = blockIdx.x * a.strips_per_wg;
    const int nl = min(a.strips_per_wg, nblocks - strip0);
    const int n0 = (blockIdx.y * NW + wave) * 128;
    const int dead = n0 < a.N ? 0 : kFar;          // wave-uniform
    const int S = gridDim.y;
    const int G = a.G;

    const rsrc_t rw = make_rsrc(a.qweight, (unsigned)((size_t)(a.K >> 3) * a.N * 4));
    const rsrc_t rs = make_rsrc(a.scales, (unsigned)((size_t)G * a.N * 2));
    const rsrc_t rz = make_rsrc(a.qzeros, (unsigned)((size_t)G * (a.N >> 3) * 4));
    const rsrc_t rdy = make_rsrc(a.dy, (unsigned)((size_t)a.M * a.N * 2));
    const int vw = dead ? 0 : (c * a.N + n0 + 8 * kk) * 4;
    const int vs = dead ? 0 : (n0 + 8 * kk) * 2;
    const int vz = dead ? 0 : ((n0 >> 3) + kk) * 4;
    const int wblock = 16 * a.N * 4;               // bytes between two output blocks (16 word-rows)

    // the chunk of dy as A operands: row-contiguous loads turned through this wavefront's own LDS (as in
    // skinny_seq_kernel); natural order, unit (4t + kk) of row c = dy[c][n0 + 32t + 8kk .. + 7]
    half8_t av[RB][NSTEP];
    {
        uint4_t xv[RB][NSTEP];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int i = 0; i < NSTEP; ++i) {
                const int vx = (min(16 * rb + 4 * i + kk, a.M - 1) * a.N + 8 * c) * 2;
                xv[rb][i] = buf_load128(rdy, vx, dead + n0 * 2);
            }
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            uint4_t* stage = reinterpret_cast<uint4_t*>(&red[rb][wave][0]);
#pragma unroll
            for (int i = 0; i < NSTEP; ++i) stage[(4 * i + kk) * 16 + (c ^ (4 * i + kk))] = xv[rb][i];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            const uint4_t* stage = reinterpret_cast<const uint4_t*>(&red[rb][wave][0]);
#pragma unroll
            for (int t = 0; t < NSTEP; ++t) av[rb][t] = __builtin_bit_cast(half8_t, stage[c * 16 + ((4 * t + kk) ^ c)]);
        }
    }
    __syncthreads();                               // red is reused by the sums below

    // one pipeline stage = SS steps of one output block
    struct Stage { uint4_t w[SS][2]; uint4_t s[SS]; uint32_t z[SS]; };
    auto load_stage = [&](Stage& st, int it) {     // it = NH * block + part, beyond the end: no traffic
        const int l = it / NH, h = it % NH;
        const int off = (dead || l >= nl) ? kFar : 0;
        const int blk = strip0 + l;
        const int g = off ? 0 : (blk << 7) / a.groupsize;
#pragma unroll
        for (int u = 0; u < SS; ++u) {
            const int t = SS * h + u;
            st.s[u] = buf_load128(rs, vs, off + g * a.N * 2 + t * 64);
            st.z[u] = buf_load32(rz, vz, off + g * (a.N >> 3) * 4 + t * 16);
        }
#pragma unroll
        for (int u = 0; u < SS; ++u) {
            const int t = SS * h + u;
            st.w[u][0] = buf_load128(rw, vw, off + blk * wblock + t * 128);
            st.w[u][1] = buf_load128(rw, vw, off + blk * wblock + t * 128 + 16);
        }
    };

    // mask in a scalar, magic number in a vector register (opaque): one and-or instruction instead of AND + OR
    uint32_t m_lo = 0x000F000Fu, g_lo = kMagic;
    asm volatile("" : "+s"(m_lo));
    asm volatile("" : "+v"(g_lo));
    float4_t acc[RB][8], corr[RB];
    auto clear_acc = [&]() {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            corr[rb] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[rb][j] = float4_t{0.f, 0.f, 0.f, 0.f};
        }
    };
    auto multiply = [&](const Stage& st, auto htag) {
        constexpr int h = decltype(htag)::value;
#pragma unroll
        for (int u = 0; u < SS; ++u) {
            constexpr int tbase = SS * h;
            const half8_t s8 = __builtin_bit_cast(half8_t, st.s[u]);
            half8_t as[RB];
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) as[rb] = av[rb][tbase + u] * s8;
            // B operand of the zero term: 1025 + z for this lane's eight columns
            const uint32_t zlo = st.z[u] & 0x0F0F0F0Fu, zhi = (st.z[u] >> 4) & 0x0F0F0F0Fu;
            const half2_t one2 = {(half_t)1.f, (half_t)1.f};
            uint32_t zb[4];
#pragma unroll
            for (int p = 0; p < 4; ++p)
                zb[p] = as_u32(as_half2(__builtin_amdgcn_perm(zhi, zlo, 0x0c040c00u + 0x00010001u * p) | kMagic) + one2);
            const half8_t zB = make_half8(zb[0], zb[1], zb[2], zb[3]);
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) corr[rb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(as[rb], zB, corr[rb], 0, 0, 0);
            // code operands: byte b of a word holds the codes of rows 2b (low nibble) and 2b + 1
            const uint32_t wd[8] = {st.w[u][0].x, st.w[u][0].y, st.w[u][0].z, st.w[u][0].w,
                                    st.w[u][1].x, st.w[u][1].y, st.w[u][1].z, st.w[u][1].w};
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                uint32_t ev[4], od[4];
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    const uint32_t sel = 0x0c000c00u | ((4u + b) << 16) | (uint32_t)b;
                    const uint32_t pb = __builtin_amdgcn_perm(wd[2 * p + 1], wd[2 * p], sel);   // byte b of columns 2p, 2p+1
                    ev[p] = (pb & m_lo) | g_lo;
                    od[p] = ((pb >> 4) & m_lo) | g_lo;
                }
                const half8_t be = make_half8(ev[0], ev[1], ev[2], ev[3]), bo = make_half8(od[0], od[1], od[2], od[3]);
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) {
                    acc[rb][2 * b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(as[rb], be, acc[rb][2 * b], 0, 0, 0);
                    acc[rb][2 * b + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(as[rb], bo, acc[rb][2 * b + 1], 0, 0, 0);
                }
            }
        }
    };
    // sums 64 outputs of the block over the wavefronts: local column lc = 4c + jj stands for output
    // 128*blk + 8*(lc / 4) + 4*hf + lc % 4; acc[rb][4*hf + jj][r] is row 16*rb + 4*kk + r
    auto finish_half = [&](int blk, int hf) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float4_t v;
#pragma unroll
                for (int jj = 0; jj < 4; ++jj) v[jj] = acc[rb][4 * hf + jj][r] - corr[rb][r];
                *reinterpret_cast<float4_t*>(&red[rb][wave][((4 * kk + r) << 6) + 4 * c]) = v;
            }
        __syncthreads();
        {
            const int e = 2 * threadIdx.x;
            const int row = e >> 6, lc = e & 63;
            const int cc = (blk << 7) + 8 * (lc >> 2) + 4 * hf + (lc & 3);
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                float v0 = 0.f, v1 = 0.f;
#pragma unroll
                for (int w = 0; w < NW; ++w) {
                    const float* rp = &red[rb][w][e];
                    v0 += rp[0];
                    v1 += rp[1];
                }
                const int m = 16 * rb + row;
                if (m < a.M) {
                    if (S == 1) {
                        const half2_t hv = {(half_t)v0, (half_t)v1};
                        *reinterpret_cast<half2_t*>(a.dx + (size_t)m * a.K + cc) = hv;
                    } else {
                        float* pp = a.part + ((size_t)blockIdx.y * a.M + m) * a.K + cc;
                        pp[0] = v0;
                        pp[1] = v1;
                    }
                }
            }
        }
        __syncthreads();
    };

    Stage buf[2];
    load_stage(buf[0], 0);
    for (int l = 0; l < nl; ++l) {
        clear_acc();
        static_for_dx<0, NH>([&](auto hc) {
            constexpr int h = decltype(hc)::value;
            load_stage(buf[(h + 1) & 1], NH * l + h + 1);      // NH is even: stage NH*l + h sits in buf[h & 1]
            __builtin_amdgcn_sched_barrier(0);
            multiply(buf[h & 1], hc);
        });
        finish_half(strip0 + l, 0);
        finish_half(strip0 + l, 1);
    }
}

// ------------------------------------------------------------------ grad-input, some hundred rows (sequential groups)
// The whole-reduction counterpart of stream_fwd_kernel for dx = dy @ W^T, with the operand scheme of skinny_dx_kernel:
// a workgroup owns one block of 128 outputs k (one quantization group) of 16*RB rows, wavefront w walks the chunks
// w, w + 8, ... of 128 columns n with its accumulators in registers (the chunk's tile of dy delivered to LDS by the
// loads themselves while the previous chunk is multiplied, words / scales / zeros one stage of SS steps ahead), and
// the eight wavefronts are summed through LDS once, at the end, into fp16 outputs: one launch, no workspace.
template <int RB, int SS>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2)))
void stream_dx_kernel(SkinnyDxArgs a) {
    constexpr int NSTEP = 4, NW = 8, NH = NSTEP / SS;
    constexpr int kFar = 0x70000000;
    __shared__ __attribute__((aligned(16))) float red[RB][NW][16 * 64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kk = lane >> 4, c = lane & 15;
    const int blk = blockIdx.x;
    const int row0 = blockIdx.z * (16 * RB);
    const int nchunks = a.N >> 7;
    const int g = (blk << 7) / a.groupsize;

    const rsrc_t rw = make_rsrc(a.qweight, (unsigned)((size_t)(a.K >> 3) * a.N * 4));
    const rsrc_t rs = make_rsrc(a.scales, (unsigned)((size_t)a.G * a.N * 2));
    const rsrc_t rz = make_rsrc(a.qzeros, (unsigned)((size_t)a.G * (a.N >> 3) * 4));
    const rsrc_t rdy = make_rsrc(a.dy, (unsigned)((size_t)a.M * a.N * 2));
    const int vw = (c * a.N + 8 * kk) * 4;
    const int vs = 16 * kk;
    const int vz = 4 * kk;
    const int wbase = blk * 16 * a.N * 4, sbase = g * a.N * 2, zbase = g * (a.N >> 3) * 4;
    // tile of dy: lane (kk, c) of load i lands at unit c of row 4i + kk and fetches unit c ^ (4i + kk) of that row (see
    // stream_fwd_kernel); rows beyond M lie beyond the buffer and read as zeros
    int vx[NSTEP];
#pragma unroll
    for (int i = 0; i < NSTEP; ++i) vx[i] = (kk * a.N + 8 * (c ^ (4 * i + kk))) * 2;
    typedef __attribute__((address_space(3))) void lds_void;
    auto fetch_tile = [&](int ch) {
        const int off = ch < nchunks ? 0 : kFar;   // past the end: no traffic
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int i = 0; i < NSTEP; ++i)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rdy, (lds_void*)(&red[rb][wave][256 * i]), 16, vx[i],
                                                         off + ((row0 + 16 * rb + 4 * i) * a.N + (ch << 7)) * 2, 0, 0);
    };
    // one pipeline stage = SS steps of 32 columns of one chunk
    struct Stage { uint4_t w[SS][2]; uint4_t s[SS]; uint32_t z[SS]; };
    auto load_stage = [&](Stage& st, int ch, int h) {
        const int off = ch < nchunks ? 0 : kFar;
        const int n0 = ch << 7;
#pragma unroll
        for (int u = 0; u < SS; ++u) {
            const int t = SS * h + u;
            st.s[u] = buf_load128(rs, vs, off + sbase + n0 * 2 + t * 64);
            st.z[u] = buf_load32(rz, vz, off + zbase + (n0 >> 1) + t * 16);
        }
#pragma unroll
        for (int u = 0; u < SS; ++u) {
            const int t = SS * h + u;
            st.w[u][0] = buf_load128_stream(rw, vw, off + wbase + n0 * 4 + t * 128);
            st.w[u][1] = buf_load128_stream(rw, vw, off + wbase + n0 * 4 + t * 128 + 16);
        }
    };

    float4_t acc[RB][8], corr[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        corr[rb] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[rb][j] = float4_t{0.f, 0.f, 0.f, 0.f};
    }
    half8_t av[RB][NSTEP];
    // mask in a scalar, magic number in a vector register (opaque): one and-or instruction instead of AND + OR
    uint32_t m_lo = 0x000F000Fu, g_lo = kMagic;
    asm volatile("" : "+s"(m_lo));
    asm volatile("" : "+v"(g_lo));
    auto multiply = [&](const Stage& st, auto htag) {
        constexpr int h = decltype(htag)::value;
#pragma unroll
        for (int u = 0; u < SS; ++u) {
            constexpr int tbase = SS * h;
            const half8_t s8 = __builtin_bit_cast(half8_t, st.s[u]);
            half8_t as[RB];
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) as[rb] = av[rb][tbase + u] * s8;
            // B operand of the zero term: 1025 + z for this lane's eight columns
            const uint32_t zlo = st.z[u] & 0x0F0F0F0Fu, zhi = (st.z[u] >> 4) & 0x0F0F0F0Fu;
            const half2_t one2 = {(half_t)1.f, (half_t)1.f};
            uint32_t zb[4];
#pragma unroll
            for (int p = 0; p < 4; ++p)
                zb[p] = as_u32(as_half2(__builtin_amdgcn_perm(zhi, zlo, 0x0c040c00u + 0x00010001u * p) | kMagic) + one2);
            const half8_t zB = make_half8(zb[0], zb[1], zb[2], zb[3]);
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) corr[rb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(as[rb], zB, corr[rb], 0, 0, 0);
            // code operands: byte b of a word holds the codes of rows 2b (low nibble) and 2b + 1
            const uint32_t wd[8] = {st.w[u][0].x, st.w[u][0].y, st.w[u][0].z, st.w[u][0].w,
                                    st.w[u][1].x, st.w[u][1].y, st.w[u][1].z, st.w[u][1].w};
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                uint32_t ev[4], od[4];
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    const uint32_t sel = 0x0c000c00u | ((4u + b) << 16) | (uint32_t)b;
                    const uint32_t pb = __builtin_amdgcn_perm(wd[2 * p + 1], wd[2 * p], sel);   // byte b of columns 2p, 2p+1
                    ev[p] = (pb & m_lo) | g_lo;
                    od[p] = ((pb >> 4) & m_lo) | g_lo;
                }
                const half8_t be = make_half8(ev[0], ev[1], ev[2], ev[3]), bo = make_half8(od[0], od[1], od[2], od[3]);
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) {
                    acc[rb][2 * b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(as[rb], be, acc[rb][2 * b], 0, 0, 0);
                    acc[rb][2 * b + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(as[rb], bo, acc[rb][2 * b + 1], 0, 0, 0);
                }
            }
        }
    };

    Stage buf[2];
    fetch_tile(wave);
    load_stage(buf[0], wave, 0);
    for (int ch = wave; ch < nchunks; ch += NW) {
        // the tile of this chunk and the first stage have landed (vmcnt 0)
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // natural order: unit (4t + kk) of row c = dy[row0 + 16 rb + c][128 ch + 32t + 8kk .. + 7]
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            const uint4_t* stage = reinterpret_cast<const uint4_t*>(&red[rb][wave][0]);
#pragma unroll
            for (int t = 0; t < NSTEP; ++t) av[rb][t] = __builtin_bit_cast(half8_t, stage[c * 16 + ((4 * t + kk) ^ c)]);
        }
        // the tile has been read (lgkmcnt 0): the next chunk of this wavefront may overwrite it
        __builtin_amdgcn_s_waitcnt(0xC07F);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_sched_barrier(0);
        fetch_tile(ch + NW);
        static_for_dx<0, NH>([&](auto hc) {
            constexpr int h = decltype(hc)::value;
            if constexpr (h + 1 < NH) load_stage(buf[(h + 1) & 1], ch, h + 1);
            else load_stage(buf[0], ch + NW, 0);                // NH is even: the next chunk starts in buf[0] again
            __builtin_amdgcn_sched_barrier(0);
            multiply(buf[h & 1], hc);
        });
    }
    // the prefetch past the last chunk may still be writing the tile: landed before the sums reuse the memory
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // sums 64 outputs of the block over the wavefronts: local column lc = 4c + jj stands for output
    // 128*blk + 8*(lc / 4) + 4*hf + lc % 4; acc[rb][4*hf + jj][r] is row row0 + 16*rb + 4*kk + r
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float4_t v;
#pragma unroll
                for (int jj = 0; jj < 4; ++jj) v[jj] = acc[rb][4 * hf + jj][r] - corr[rb][r];
                *reinterpret_cast<float4_t*>(&red[rb][wave][((4 * kk + r) << 6) + 4 * c]) = v;
            }
        __syncthreads();
        {
            const int e = 2 * threadIdx.x;
            const int row = e >> 6, lc = e & 63;
            const int cc = (blk << 7) + 8 * (lc >> 2) + 4 * hf + (lc & 3);
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                float v0 = 0.f, v1 = 0.f;
#pragma unroll
                for (int w = 0; w < NW; ++w) {
                    const float* rp = &red[rb][w][e];
                    v0 += rp[0];
                    v1 += rp[1];
                }
                const int m = row0 + 16 * rb + row;
                if (m < a.M) {
                    const half2_t hv = {(half_t)v0, (half_t)v1};
                    *reinterpret_cast<half2_t*>(a.dx + (size_t)m * a.K + cc) = hv;
                }
            }
        }
        __syncthreads();
    }
}

// ------------------------------------------------------------------ act-order (per-row groups)
template <int NSTEP>
__global__ __launch_bounds__(512) void gemv_gidx_kernel(GemvArgs a) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nwaves = blockDim.x >> 6;
    const int kk = lane >> 4, c = lane & 15;
    const int n0 = blockIdx.x * kColsPerWave;
    const int k0 = (blockIdx.y * nwaves + wave) * (32 * NSTEP);

    float4_t yacc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) yacc[j] = float4_t{0.f, 0.f, 0.f, 0.f};

    if (k0 < a.K) {
        const int ncol8 = a.N >> 3;
        const int col = n0 + 4 * c;
        const int zshift = (c & 1) * 16;
        uint4_t wv[NSTEP], xv[NSTEP], ga[NSTEP], gb[NSTEP];
        const uint32_t* wp = a.qweight + (size_t)((k0 >> 3) + kk) * a.N + col;
        const half_t* xp = a.x + (size_t)min(c, a.M - 1) * a.K + k0 + 8 * kk;
        const int32_t* gp = a.g_idx + k0 + 8 * kk;
#pragma unroll
        for (int t = 0; t < NSTEP; ++t) {
            ga[t] = *reinterpret_cast<const uint4_t*>(gp + 32 * t);
            gb[t] = *reinterpret_cast<const uint4_t*>(gp + 32 * t + 4);
        }
#pragma unroll
        for (int t = 0; t < NSTEP; ++t) {
            wv[t] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(wp + (size_t)(4 * t) * a.N));
            xv[t] = *reinterpret_cast<const uint4_t*>(xp + 32 * t);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < NSTEP; ++t) {
            const uint32_t g[8] = {ga[t].x, ga[t].y, ga[t].z, ga[t].w, gb[t].x, gb[t].y, gb[t].z, gb[t].w};
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
    gemv_finish(a, yacc, n0, wave, nwaves, kk, c, gridDim.y);
}

}  // namespace q4

extern "C" size_t q4_gemv_workspace_bytes(int M, int K, int N) {
    (void)K;
    if (M < 1 || N < 1) return 0;
    return (size_t)M * (size_t)N * sizeof(unsigned long long);
}

template <int NSTEP>
static void launch_seq(const q4::GemvPlan& p, dim3 grid, dim3 block, size_t lds, hipStream_t stream, const q4::GemvArgs& a) {
    using namespace q4;
    switch (p.gsteps) {
        case 0: hipLaunchKernelGGL((gemv_seq_kernel<NSTEP, 0>), grid, block, lds, stream, a); break;
        case 1: if constexpr (NSTEP > 1) hipLaunchKernelGGL((gemv_seq_kernel<NSTEP, 1>), grid, block, lds, stream, a); break;
        case 2: if constexpr (NSTEP > 2) hipLaunchKernelGGL((gemv_seq_kernel<NSTEP, 2>), grid, block, lds, stream, a); break;
        case 4: if constexpr (NSTEP > 4) hipLaunchKernelGGL((gemv_seq_kernel<NSTEP, 4>), grid, block, lds, stream, a); break;
        case 8: if constexpr (NSTEP > 8) hipLaunchKernelGGL((gemv_seq_kernel<NSTEP, 8>), grid, block, lds, stream, a); break;
    }
}

// Shapes q4_gemv_sorted_f16 takes: up to 4 rows whose activations (plus 4 KB per row of staging) fit in 64 KB of LDS.
extern "C" int q4_gemv_sorted_applicable(int M, int K) {
    return M >= 1 && M <= 4 && K >= 1024 && (size_t)M * ((size_t)K * 2 + 4096) <= 65536;   // K >= 1024: 8 wavefronts
}

template <int NSTEP>
static void launch_seq_perm(const q4::GemvPlan& p, dim3 grid, dim3 block, size_t lds, hipStream_t stream, const q4::GemvArgs& a) {
    using namespace q4;
    switch (p.gsteps) {
        case 0: hipLaunchKernelGGL((gemv_seq_perm_kernel<NSTEP, 0>), grid, block, lds, stream, a); break;
        case 1: if constexpr (NSTEP > 1) hipLaunchKernelGGL((gemv_seq_perm_kernel<NSTEP, 1>), grid, block, lds, stream, a); break;
        case 2: if constexpr (NSTEP > 2) hipLaunchKernelGGL((gemv_seq_perm_kernel<NSTEP, 2>), grid, block, lds, stream, a); break;
    }
}

// `perm` != null: the packed rows are sorted by group and x is gathered through perm inside the kernel
// (sequential groups only, M <= 4).
extern "C" int q4_launch_gemv(const void* x, const int32_t* qweight, const int32_t* qzeros, const void* scales,
                              const int32_t* g_idx, const int32_t* perm, int groupsize, void* y, int accumulate,
                              int M, int K, int N, int G, void* workspace, hipStream_t stream) {
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
    a.M = M; a.K = K; a.N = N; a.G = G;
    a.acc64 = reinterpret_cast<unsigned long long*>(workspace);
    a.perm = perm;
    a.v1_zeros = nullptr;

    const bool seq = (g_idx == nullptr);
    const GemvPlan p = plan_gemv(K, N, groupsize, seq, 4);
    const dim3 grid(N / kColsPerWave, p.splits);
    const dim3 block(64 * p.waves);
    const size_t lds = (size_t)p.waves * M * 64 * sizeof(float);
    if (perm) {
        // + the operand tile and the activation rows; q4_gemv_sorted_applicable() keeps this within 64 KB
        const size_t lds_x = lds + (size_t)M * p.waves * 32 * p.nstep * sizeof(half_t) + (size_t)M * K * sizeof(half_t);
        if (!seq || M > 4 || lds_x > 65536 || (size_t)M * K / 8 > (size_t)8 * block.x) return -2;
        switch (p.nstep) {
            case 4: launch_seq_perm<4>(p, grid, block, lds_x, stream, a); break;
            case 2: launch_seq_perm<2>(p, grid, block, lds_x, stream, a); break;
            default: launch_seq_perm<1>(p, grid, block, lds_x, stream, a); break;
        }
    } else if (seq) {
        switch (p.nstep) {
            case 16: launch_seq<16>(p, grid, block, lds, stream, a); break;
            case 8: launch_seq<8>(p, grid, block, lds, stream, a); break;
            case 4: launch_seq<4>(p, grid, block, lds, stream, a); break;
            case 2: launch_seq<2>(p, grid, block, lds, stream, a); break;
            default: launch_seq<1>(p, grid, block, lds, stream, a); break;
        }
    } else {
        switch (p.nstep) {
            case 4: hipLaunchKernelGGL(gemv_gidx_kernel<4>, grid, block, lds, stream, a); break;
            case 2: hipLaunchKernelGGL(gemv_gidx_kernel<2>, grid, block, lds, stream, a); break;
            default: hipLaunchKernelGGL(gemv_gidx_kernel<1>, grid, block, lds, stream, a); break;
        }
    }
    return hipGetLastError() == hipSuccess ? 0 : -4;
}


template <int NSTEP>
static void launch_seq_group(const q4::GemvPlan& p, dim3 grid, dim3 block, size_t lds, hipStream_t stream,
                             const q4::GemvGroupArgs& g) {
    using namespace q4;
    switch (p.gsteps) {
        case 0: hipLaunchKernelGGL((gemv_seq_group_kernel<NSTEP, 0>), grid, block, lds, stream, g); break;
        case 1: if constexpr (NSTEP > 1) hipLaunchKernelGGL((gemv_seq_group_kernel<NSTEP, 1>), grid, block, lds, stream, g); break;
        case 2: if constexpr (NSTEP > 2) hipLaunchKernelGGL((gemv_seq_group_kernel<NSTEP, 2>), grid, block, lds, stream, g); break;
    }
}

// n layers (1..4) sharing M, K and the group size (sequential groups); layer i: x[i], packed tensors, y[i], N[i];
// its accumulators start at workspace + 8*M*(N[0] + .. + N[i-1]).
extern "C" int q4_launch_gemv_group(int n, const void* const* x, const int32_t* const* qweight,
                                    const int32_t* const* qzeros, const void* const* scales, void* const* y,
                                    const int* N, int groupsize, int accumulate, int M, int K, int G,
                                    void* workspace, hipStream_t stream) {
    using namespace q4;
    GemvGroupArgs g;
    int strips = 0;
    size_t ws_off = 0;
    for (int i = 0; i < kMaxGroup; ++i) {
        const int j = i < n ? i : n - 1;              // unused slots repeat the last layer (never selected)
        GemvArgs& a = g.layer[i];
        a.x = reinterpret_cast<const half_t*>(x[j]);
        a.qweight = reinterpret_cast<const uint32_t*>(qweight[j]);
        a.qzeros = reinterpret_cast<const uint32_t*>(qzeros[j]);
        a.scales = reinterpret_cast<const half_t*>(scales[j]);
        a.g_idx = nullptr;
        a.groupsize = groupsize;
        a.y = reinterpret_cast<half_t*>(y[j]);
        a.accumulate = accumulate;
        a.M = M; a.K = K; a.N = N[j]; a.G = G;
        a.acc64 = reinterpret_cast<unsigned long long*>(workspace) + ws_off;
        a.perm = nullptr;
        a.v1_zeros = nullptr;
        if (i < n) {
            strips += N[i] / kColsPerWave;
            ws_off += (size_t)M * N[i];
            g.strip_end[i] = strips;
        } else {
            g.strip_end[i] = 0x7fffffff;
        }
    }
    const GemvPlan p = plan_gemv(K, N[0], groupsize, true, 4);      // the plan does not depend on N
    const dim3 grid(strips, p.splits), block(64 * p.waves);
    const size_t lds = (size_t)p.waves * M * 64 * sizeof(float);
    switch (p.nstep) {
        case 4: launch_seq_group<4>(p, grid, block, lds, stream, g); break;
        case 2: launch_seq_group<2>(p, grid, block, lds, stream, g); break;
        default: launch_seq_group<1>(p, grid, block, lds, stream, g); break;
    }
    return hipGetLastError() == hipSuccess ? 0 : -4;
}

// v1 layout: scales and zeros are fp16 [N]; one group spanning K.
extern "C" int q4_launch_gemv_v1(const void* x, const int32_t* qweight, const void* scales, const void* zeros, void* y,
                                 int accumulate, int M, int K, int N, void* workspace, hipStream_t stream) {
    using namespace q4;
    GemvArgs a;
    a.x = reinterpret_cast<const half_t*>(x);
    a.qweight = reinterpret_cast<const uint32_t*>(qweight);
    a.qzeros = nullptr;
    a.scales = reinterpret_cast<const half_t*>(scales);
    a.g_idx = nullptr;
    a.groupsize = K;
    a.y = reinterpret_cast<half_t*>(y);
    a.accumulate = accumulate;
    a.M = M; a.K = K; a.N = N; a.G = 1;
    a.acc64 = reinterpret_cast<unsigned long long*>(workspace);
    a.perm = nullptr;
    a.v1_zeros = reinterpret_cast<const half_t*>(zeros);
    const GemvPlan p = plan_gemv(K, N, K, true, 4);
    const dim3 grid(N / kColsPerWave, p.splits), block(64 * p.waves);
    const size_t lds = (size_t)p.waves * M * 64 * sizeof(float);
    switch (p.nstep) {                                       // one group: gsteps is always 0
        case 4: hipLaunchKernelGGL((gemv_seq_kernel<4, 0, true>), grid, block, lds, stream, a); break;
        case 2: hipLaunchKernelGGL((gemv_seq_kernel<2, 0, true>), grid, block, lds, stream, a); break;
        default: hipLaunchKernelGGL((gemv_seq_kernel<1, 0, true>), grid, block, lds, stream, a); break;
    }
    return hipGetLastError() == hipSuccess ? 0 : -4;
}

extern "C" int q4_launch_splitk_reduce(const float* part, void* out, long total, int splits, hipStream_t stream);

// Shapes the skinny kernel takes: 17..64 rows, sequential groups that are multiples of 128 rows.
extern "C" int q4_skinny_applicable(int M, int K, int N, int groupsize, int has_gidx) {
    return M > 16 && M <= 64 && !has_gidx && groupsize > 0 && groupsize % 128 == 0 && K % 128 == 0 && N % 64 == 0;
}

static int skinny_splits(int K) {
    const int chunks = K / 128;
    return (chunks + 7) / 8;                      // 8 wavefronts per workgroup, one chunk each
}

extern "C" size_t q4_skinny_workspace(int M, int K, int N) {
    const int S = skinny_splits(K);
    return S > 1 ? (size_t)S * (size_t)M * (size_t)N * sizeof(float) : 0;
}

extern "C" int q4_launch_skinny(const void* x, const int32_t* qweight, const int32_t* qzeros, const void* scales,
                                int groupsize, const void* bias, void* y, int M, int K, int N, int G,
                                void* workspace, hipStream_t stream) {
    using namespace q4;
    SkinnyArgs a;
    a.x = reinterpret_cast<const half_t*>(x);
    a.qweight = reinterpret_cast<const uint32_t*>(qweight);
    a.qzeros = reinterpret_cast<const uint32_t*>(qzeros);
    a.scales = reinterpret_cast<const half_t*>(scales);
    a.bias = reinterpret_cast<const half_t*>(bias);
    a.groupsize = groupsize;
    a.y = reinterpret_cast<half_t*>(y);
    a.part = reinterpret_cast<float*>(workspace);
    a.M = M; a.K = K; a.N = N; a.G = G;
    const int S = skinny_splits(K);
    const int strips = N / kColsPerWave;
    // neighbouring strips per workgroup: enough for the whole grid to be resident at once (two workgroups
    // per compute unit fit with two row blocks, one with more), at most 4
    const int slots = M <= 32 ? 512 : 256;
    int L = (strips * S + slots - 1) / slots;
    L = L < 1 ? 1 : (L > 4 ? 4 : L);
    a.strips_per_wg = L;
    const dim3 grid((strips + L - 1) / L, S), block(512);    // wavefronts past the end of K read zeros
    if (M <= 32) hipLaunchKernelGGL(skinny_seq_kernel<2>, grid, block, 0, stream, a);
    else if (M <= 48) hipLaunchKernelGGL(skinny_seq_kernel<3>, grid, block, 0, stream, a);
    else hipLaunchKernelGGL(skinny_seq_kernel<4>, grid, block, 0, stream, a);
    if (hipGetLastError() != hipSuccess) return -4;
    if (S > 1) return q4_launch_splitk_reduce(a.part, y, (long)M * N, S, stream);
    return 0;
}

// Shapes the whole-reduction streaming kernel takes: more than 64 rows (from 17 rows on wide outputs), sequential groups
// that are multiples of 128 rows, and an output small enough for ONE round of workgroups (at most one per CU): the kernel is bound per CU (the
// vector-ALU work of the operand build, the activation tiles every wavefront pulls), so a second round costs as much as
// the first, while the tiled kernel only gets better with more tiles (measured on 4096 x 4096, 65..256 rows: 10.2-16.1 us
// against 16.1-24.4 us; 2048 x 2048, 65..512 rows: 7-10.6 against 12.3-22.3 us; 11008 -> 4096, up to 192 rows: 22-31
// against 22-34 us; 4096 -> 11008 never fits one round).
// Row blocks of 32, 48 or 64 rows: the smallest that fits (more workgroups, fewer idle CUs).
static int stream_fwd_row_blocks(int M, int N) {
    const int strips = N / q4::kColsPerWave;
    for (int rb = 2; rb <= 4; ++rb)
        if (strips * ((M + 16 * rb - 1) / (16 * rb)) <= 256) return rb;
    return 0;
}
extern "C" int q4_stream_fwd_applicable(int M, int K, int N, int groupsize, int has_gidx) {
    if (!(M > 16 && M <= 512 && !has_gidx && groupsize > 0 && groupsize % 128 == 0 && K % 128 == 0 && N % 64 == 0))
        return 0;
    // up to 64 rows there is one row block, i.e. one workgroup per strip: worth it from 128 strips on, where it beats
    // the kernel with the split reduction and the second launch (4096 -> 11008 at 17..64 rows: 9.7-14.7 against
    // 14.5-18.1 us, 5120 -> 13824: 11.9-17.7 against 18.5-35.2 us; at 64 strips it loses, 4096 x 4096: 9.7-10.4 against 8.7-10.8 us)
    if (M <= 64 && N < 8192) return 0;
    if (K > 65536 || N > 65536 || (long)K * N > (1L << 28)) return 0;      // 32-bit byte offsets, far offset included
    // very long reductions with the larger row blocks: level with the tiled kernel or just behind (13824 -> 5120)
    const int rb = stream_fwd_row_blocks(M, N);
    return rb == 2 || (rb > 2 && K <= 12288);
}

extern "C" int q4_launch_stream_fwd(const void* x, const int32_t* qweight, const int32_t* qzeros, const void* scales,
                                    int groupsize, const void* bias, void* y, int M, int K, int N, int G,
                                    hipStream_t stream) {
    using namespace q4;
    SkinnyArgs a;
    a.x = reinterpret_cast<const half_t*>(x);
    a.qweight = reinterpret_cast<const uint32_t*>(qweight);
    a.qzeros = reinterpret_cast<const uint32_t*>(qzeros);
    a.scales = reinterpret_cast<const half_t*>(scales);
    a.bias = reinterpret_cast<const half_t*>(bias);
    a.groupsize = groupsize;
    a.y = reinterpret_cast<half_t*>(y);
    a.part = nullptr;
    a.M = M; a.K = K; a.N = N; a.G = G;
    a.strips_per_wg = 1;
    const int strips = N / kColsPerWave;
    const int rb = stream_fwd_row_blocks(M, N);
    if (rb == 0) return -2;
    const dim3 grid(strips, 1, (M + 16 * rb - 1) / (16 * rb)), block(512);
    if (rb == 2) hipLaunchKernelGGL(stream_fwd_kernel<2>, grid, block, 0, stream, a);
    else if (rb == 3) hipLaunchKernelGGL(stream_fwd_kernel<3>, grid, block, 0, stream, a);
    else hipLaunchKernelGGL(stream_fwd_kernel<4>, grid, block, 0, stream, a);
    return hipGetLastError() == hipSuccess ? 0 : -4;
}

// Shapes the whole-reduction grad-input kernel takes: as q4_stream_fwd_applicable, with blocks of 128 outputs and row
// blocks of 32 or 48 rows (the accumulators of 64 rows do not fit the registers); below 49 rows skinny_dx_kernel is
// faster on every shape measured (e.g. 8192 x 8192 at 17..48 rows: 15-18 against 28-30 us).  Measured, 49..256 rows: 4096 x 4096
// 15.5-17.3 against 15.5-24.8 us, 2048 x 2048 10 against 12-18.5 us, 4096 outputs over 1024 columns 7.6 against 11-18 us,
// 11008 outputs over 4096 columns (up to 96 rows) 18-21 against 28-32 us.
static int stream_dx_row_blocks(int M, int K) {
    const int blocks = K / 128;
    for (int rb = 2; rb <= 3; ++rb)
        if (blocks * ((M + 16 * rb - 1) / (16 * rb)) <= 256) return rb;
    return 0;
}
extern "C" int q4_stream_dx_applicable(int M, int K, int N, int groupsize, int has_gidx) {
    if (!(M > 48 && M <= 512 && !has_gidx && groupsize > 0 && groupsize % 128 == 0 && K % 128 == 0 && N % 128 == 0))
        return 0;
    if (K > 65536 || N > 65536 || (long)K * N > (1L << 28)) return 0;      // 32-bit byte offsets, far offset included
    // a workgroup walks the whole reduction alone: with a long reduction and few output blocks (4096 outputs over 11008
    // columns: 38-42 us against 24-38 us) the tiled kernel with its split reduction is faster
    return N <= 2 * K && stream_dx_row_blocks(M, K) != 0;
}

extern "C" int q4_launch_stream_dx(const void* dy, const int32_t* qweight, const int32_t* qzeros, const void* scales,
                                   int groupsize, void* dx, int M, int K, int N, int G, hipStream_t stream) {
    using namespace q4;
    SkinnyDxArgs a;
    a.dy = reinterpret_cast<const half_t*>(dy);
    a.qweight = reinterpret_cast<const uint32_t*>(qweight);
    a.qzeros = reinterpret_cast<const uint32_t*>(qzeros);
    a.scales = reinterpret_cast<const half_t*>(scales);
    a.groupsize = groupsize;
    a.dx = reinterpret_cast<half_t*>(dx);
    a.part = nullptr;
    a.M = M; a.K = K; a.N = N; a.G = G;
    a.strips_per_wg = 1;
    const int rb = stream_dx_row_blocks(M, K);
    if (rb == 0) return -2;
    const dim3 grid(K / 128, 1, (M + 16 * rb - 1) / (16 * rb)), block(512);
    if (rb == 2) hipLaunchKernelGGL((stream_dx_kernel<2, 2>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((stream_dx_kernel<3, 1>), grid, block, 0, stream, a);
    return hipGetLastError() == hipSuccess ? 0 : -4;
}

// Shapes the streaming grad-input kernel takes: 17..48 rows, sequential groups that are multiples of 128 rows.
extern "C" int q4_skinny_dx_applicable(int M, int K, int N, int groupsize, int has_gidx) {
    return M > 16 && M <= 48 && !has_gidx && groupsize > 0 && groupsize % 128 == 0 && K % 128 == 0 &&
           N % 128 == 0;
}

static int skinny_dx_splits(int N) {
    return (N / 128 + 7) / 8;                     // 8 wavefronts per workgroup, one chunk of 128 columns each
}

extern "C" size_t q4_skinny_dx_workspace(int M, int K, int N) {
    const int S = skinny_dx_splits(N);
    return S > 1 ? (size_t)S * (size_t)M * (size_t)K * sizeof(float) : 0;
}

extern "C" int q4_launch_skinny_dx(const void* dy, const int32_t* qweight, const int32_t* qzeros, const void* scales,
                                   int groupsize, void* dx, int M, int K, int N, int G, void* workspace,
                                   hipStream_t stream) {
    using namespace q4;
    SkinnyDxArgs a;
    a.dy = reinterpret_cast<const half_t*>(dy);
    a.qweight = reinterpret_cast<const uint32_t*>(qweight);
    a.qzeros = reinterpret_cast<const uint32_t*>(qzeros);
    a.scales = reinterpret_cast<const half_t*>(scales);
    a.groupsize = groupsize;
    a.dx = reinterpret_cast<half_t*>(dx);
    a.part = reinterpret_cast<float*>(workspace);
    a.M = M; a.K = K; a.N = N; a.G = G;
    const int S = skinny_dx_splits(N);
    const int blocks = K / 128;
    const int slots = 256;                        // one workgroup per compute unit (register budget)
    int L = (blocks * S + slots - 1) / slots;
    L = L < 1 ? 1 : (L > 4 ? 4 : L);
    a.strips_per_wg = L;
    const dim3 grid((blocks + L - 1) / L, S), block(512);     // wavefronts past the end of N read zeros
    if (M <= 32) hipLaunchKernelGGL((skinny_dx_kernel<2, 2>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((skinny_dx_kernel<3, 1>), grid, block, 0, stream, a);   // a fourth row block would not fit the registers
    if (hipGetLastError() != hipSuccess) return -4;
    if (S > 1) return q4_launch_splitk_reduce(a.part, dx, (long)M * K, S, stream);
    return 0;
}

// ------------------------------------------------------------------ split-K accumulators owned by the library
// For callers that cannot allocate (q4_gemv_noalloc_f16): the [M, N] 64-bit accumulators live in a file-scope
// device array instead of a caller workspace.  Every device that loads this library holds its own copy at its
// own address; host code must never hand the array's NAME to a kernel (on the host it is only a stand-in
// symbol), so the device address is looked up once per device and kept.
namespace q4 {
constexpr size_t kNoAllocWords = (size_t)16 * 32768;          // M * N <= 524 288 accumulators = 4 MiB per device
static __device__ __align__(256) unsigned long long noalloc_scratch[kNoAllocWords];

__global__ __launch_bounds__(256) void zero_words_kernel(unsigned long long* p, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0ull;
}
}  // namespace q4

extern "C" size_t q4_noalloc_scratch_bytes(void) { return q4::kNoAllocWords * sizeof(unsigned long long); }

// Device address of the array on the CURRENT device (looked up on the first call per device), or null with
// *err set to the HIP error.
extern "C" void* q4_noalloc_scratch_ptr(int* err) {
    constexpr int kMaxDevices = 64;
    static void* volatile ptrs[kMaxDevices];
    *err = 0;
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) { *err = e != hipSuccess ? (int)e : -1; return nullptr; }
    void* p = ptrs[dev];
    if (p) return p;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(q4::noalloc_scratch));
    if (e != hipSuccess || !p) { *err = e != hipSuccess ? (int)e : -1; return nullptr; }
    ptrs[dev] = p;                                              // racing first calls store the same address
    return p;
}

// Zeroes the first `words` accumulators with a small kernel (a fill kernel, not a memset node, so that the call
// may be recorded into a HIP graph).
extern "C" int q4_launch_zero_words(void* p, size_t words, hipStream_t stream) {
    if (words == 0) return 0;
    hipLaunchKernelGGL(q4::zero_words_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, stream,
                       reinterpret_cast<unsigned long long*>(p), (int)words);
    return hipGetLastError() == hipSuccess ? 0 : -4;
}
