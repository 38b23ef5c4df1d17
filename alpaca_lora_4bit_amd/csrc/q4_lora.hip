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
#include <stdlib.h>

namespace q4 {

constexpr int kFarOffset = 0x70000000;      // beyond any buffer accepted here: such loads return zero, no traffic

__device__ __forceinline__ half8_t to_half8(float4_t a, float4_t b) {
    half8_t r;
#pragma unroll
    for (int e = 0; e < 4; ++e) { r[e] = (half_t)a[e]; r[4 + e] = (half_t)b[e]; }
    return r;
}

// ---- down projection -------------------------------------------------------------------
// Workgroup = 16 wavefronts on 16 rows; wavefront w multiplies the C/16-wide slice w of those rows
// with v_mfma_f32_16x16x32_f16 (A operand = 16 rows x 32 columns of `in`, B operand = the same 32
// columns of up to 16 rows of W); the partial 16 x 16 results are added through LDS.  R <= 64 is
// handled as RB = ceil(R/16) column blocks.
// All loads are buffer loads whose out-of-range lanes (rows past M, adapter rows past R, steps past
// the wavefront's slice) return zero: no branch sits between the loads of a batch of UN steps, so they
// are all in flight together.  Three ways to fetch W[j][c] -> the B operand (8 consecutive c per lane):
//   kRowsT c contiguous in memory (lora_A.weight [R, C]), R <= 16: each adapter row's 256-column piece is
//          loaded as one fully coalesced instruction (4 values per lane), converted, and passed to the
//          operand layout through a wavefront-private LDS tile
//   kCols  j contiguous in memory (lora_B.weight [C, R] seen as W = B^T), R <= 16, R % 4 == 0: groups of 4
//          adapter rows are loaded coalesced and transposed through the same LDS tile
//   kRows  c contiguous, any R <= 64: one or two 16-byte loads per lane and step straight into the operand
//   kAny   arbitrary strides: eight scalar loads per lane and step
enum WLayout { kRows = 0, kCols = 1, kAny = 2, kRowsT = 3 };
constexpr int kDownWaves = 16;

template <int RB, int WL, bool F32, int RQ>   // RQ: ceil(R/4) for kCols / kRowsT, else unused
__global__ __launch_bounds__(64 * kDownWaves) void lora_down_kernel(const half_t* __restrict__ in,
                                                                    const void* __restrict__ w, int w_sr, int w_sc,
                                                                    half_t* __restrict__ out, int M, int C, int R,
                                                                    int rows, DropArgs drop) {
    constexpr int NW = kDownWaves;
    constexpr int UN = WL == kAny ? (RB == 1 ? 4 : RB == 2 ? 2 : 1) : (RB == 1 ? 8 : 4);   // steps whose loads are issued together
    constexpr int ES = F32 ? 4 : 2;
    constexpr int TRW = UN * 32 + 8;                            // padded row of the transposition tile (halves)
    __shared__ float red[NW][RB][256];
    constexpr bool kStaged = WL == kCols || WL == kRowsT;
    __shared__ __attribute__((aligned(16))) half_t tr[kStaged ? NW : 1][16][kStaged ? TRW : 8];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kk = lane >> 4, c = lane & 15;
    const int m0 = blockIdx.x * rows;                           // rows = 16, 8 or 4: operand rows past it read as zero
    const int steps = C / 32;                                   // C is a multiple of 32
    const int s_begin = (steps * wave) / NW, s_end = (steps * (wave + 1)) / NW;
    const rsrc_t rs_in = make_rsrc(in + (size_t)m0 * C, (unsigned)min(rows, M - m0) * (unsigned)C * 2u);
    const rsrc_t rs_w = make_rsrc(w, ((unsigned)(R - 1) * (unsigned)w_sr + (unsigned)(C - 1) * (unsigned)w_sc + 1u) * ES);
    const int voff_in = (c * C + 8 * kk) * 2;
    float4_t acc[RB];
#pragma unroll
    for (int b = 0; b < RB; ++b) acc[b] = float4_t{0.f, 0.f, 0.f, 0.f};
    // dropout of `in` (uniform branch): this lane's operand is row m0 + c, columns 32*s + 8*kk .. + 7 of step s
    const uint32_t drop_key = drop_row_key(drop, (uint32_t)(m0 + c));
    const uint32_t thr_pair = drop.thr15 | (drop.thr15 << 16);

    for (int s0 = s_begin; s0 < s_end; s0 += UN) {
        uint4_t av[UN];
        half8_t bv[UN][RB];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int s = s0 + u;
            av[u] = buf_load128(rs_in, voff_in, s < s_end ? s * 64 : kFarOffset);
        }
        if constexpr (WL == kRows) {
            uint4_t raw[UN][RB][F32 ? 2 : 1];
#pragma unroll
            for (int u = 0; u < UN; ++u) {
                const int s = s0 + u;
                const int soff = s < s_end ? s * 32 * ES : kFarOffset;
#pragma unroll
                for (int b = 0; b < RB; ++b) {
                    const int j = 16 * b + c;
                    const int voff = j < R ? (j * w_sr + 8 * kk) * ES : kFarOffset;
                    raw[u][b][0] = buf_load128(rs_w, voff, soff);
                    if constexpr (F32) raw[u][b][1] = buf_load128(rs_w, voff + 16, soff);
                }
            }
#pragma unroll
            for (int u = 0; u < UN; ++u)
#pragma unroll
                for (int b = 0; b < RB; ++b) {
                    if constexpr (F32) bv[u][b] = to_half8(__builtin_bit_cast(float4_t, raw[u][b][0]), __builtin_bit_cast(float4_t, raw[u][b][1]));
                    else bv[u][b] = __builtin_bit_cast(half8_t, raw[u][b][0]);
                }
        } else if constexpr (kStaged) {
            // fill the tile tr[j][column within the batch] with fp16 values of W
            if constexpr (WL == kCols) {
                // UN*32 columns x RQ groups of 4 adapter rows, 64 items per load instruction
                constexpr int NT = UN * 32 * RQ / 64;
                uint4_t raw[NT];
                const int soff = s0 * 32 * w_sc * ES;
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const int i = lane + 64 * t, cl = i / RQ, q = i - cl * RQ;
                    const int voff = (s0 * 32 + cl) < s_end * 32 ? (cl * w_sc + 4 * q) * ES : kFarOffset;
                    if constexpr (F32) raw[t] = buf_load128(rs_w, voff, soff);
                    else { const uint2_t v = buf_load64(rs_w, voff, soff); raw[t] = uint4_t{v.x, v.y, 0u, 0u}; }
                }
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const int i = lane + 64 * t, cl = i / RQ, q = i - cl * RQ;
                    half_t h[4];
                    if constexpr (F32) {
                        const float4_t f = __builtin_bit_cast(float4_t, raw[t]);
#pragma unroll
                        for (int e = 0; e < 4; ++e) h[e] = (half_t)f[e];
                    } else {
                        const half2_t lo = as_half2(raw[t].x), hi = as_half2(raw[t].y);
                        h[0] = lo[0]; h[1] = lo[1]; h[2] = hi[0]; h[3] = hi[1];
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) tr[wave][4 * q + e][cl] = h[e];
                }
            } else {
                // 4*RQ adapter rows; per row the batch's UN*32 columns, 4 per lane
                constexpr int NL = UN * 32 / 256;                 // load instructions per row (1 for UN = 8)
                static_assert(NL >= 1, "a batch must cover at least 256 columns");
                uint4_t raw[4 * RQ][NL];
                const int soff = s0 * 32 * ES;
#pragma unroll
                for (int j = 0; j < 4 * RQ; ++j)
#pragma unroll
                    for (int t = 0; t < NL; ++t) {
                        const int cl = 4 * (lane + 64 * t);
                        const int voff = (j < R && (s0 * 32 + cl) < s_end * 32) ? (j * w_sr + cl) * ES : kFarOffset;
                        if constexpr (F32) raw[j][t] = buf_load128(rs_w, voff, soff);
                        else { const uint2_t v = buf_load64(rs_w, voff, soff); raw[j][t] = uint4_t{v.x, v.y, 0u, 0u}; }
                    }
#pragma unroll
                for (int j = 0; j < 4 * RQ; ++j)
#pragma unroll
                    for (int t = 0; t < NL; ++t) {
                        const int cl = 4 * (lane + 64 * t);
                        uint2_t packed;
                        if constexpr (F32) {
                            const float4_t f = __builtin_bit_cast(float4_t, raw[j][t]);
                            const half2_t lo = {(half_t)f[0], (half_t)f[1]}, hi = {(half_t)f[2], (half_t)f[3]};
                            packed = uint2_t{as_u32(lo), as_u32(hi)};
                        } else {
                            packed = uint2_t{raw[j][t].x, raw[j][t].y};
                        }
                        *reinterpret_cast<uint2_t*>(&tr[wave][j][cl]) = packed;
                    }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int u = 0; u < UN; ++u) {
                const half8_t v = *reinterpret_cast<const half8_t*>(&tr[wave][c][32 * u + 8 * kk]);
#pragma unroll
                for (int e = 0; e < 8; ++e) bv[u][0][e] = c < 4 * RQ ? v[e] : (half_t)0.f;   // rows past R were never written
            }
            __builtin_amdgcn_wave_barrier();
        } else {
            uint32_t raw[UN][RB][8];
#pragma unroll
            for (int u = 0; u < UN; ++u) {
                const int s = s0 + u;
                const int soff = s < s_end ? s * 32 * w_sc * ES : kFarOffset;
#pragma unroll
                for (int b = 0; b < RB; ++b) {
                    const int j = 16 * b + c;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const int voff = j < R ? (j * w_sr + (8 * kk + e) * w_sc) * ES : kFarOffset;
                        raw[u][b][e] = F32 ? buf_load32(rs_w, voff, soff) : buf_load16(rs_w, voff, soff);
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < UN; ++u)
#pragma unroll
                for (int b = 0; b < RB; ++b)
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        bv[u][b][e] = F32 ? (half_t)__builtin_bit_cast(float, raw[u][b][e])
                                          : __builtin_bit_cast(half_t, (uint16_t)raw[u][b][e]);
        }
        // dropout of `in`, after every load of the batch has been issued (steps past the slice hold zeros anyway)
        if (drop.thr15) {
#pragma unroll
            for (int u = 0; u < UN; ++u) {
                const uint32_t pair0 = (uint32_t)(s0 + u) * 16u + 4u * kk;
                av[u].x &= drop_keep_mask(drop_word(drop, drop_key, pair0), thr_pair);
                av[u].y &= drop_keep_mask(drop_word(drop, drop_key, pair0 + 1), thr_pair);
                av[u].z &= drop_keep_mask(drop_word(drop, drop_key, pair0 + 2), thr_pair);
                av[u].w &= drop_keep_mask(drop_word(drop, drop_key, pair0 + 3), thr_pair);
            }
        }
        // steps past the slice were loaded as zeros: they add nothing
#pragma unroll
        for (int u = 0; u < UN; ++u)
#pragma unroll
            for (int b = 0; b < RB; ++b)
                acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, av[u]), bv[u][b], acc[b], 0, 0, 0);
    }
    // acc[b][r]: row 4*kk + r, column 16*b + c
#pragma unroll
    for (int b = 0; b < RB; ++b)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[wave][b][(4 * kk + r) * 16 + c] = acc[b][r];
    __syncthreads();
    for (int e = threadIdx.x; e < RB * 256; e += 64 * NW) {
        const int b = e >> 8, i = e & 255;
        float v = 0.f;
#pragma unroll
        for (int wv = 0; wv < NW; ++wv) v += red[wv][b][i];
        const int m = m0 + (i >> 4), j = 16 * b + (i & 15);
        if ((i >> 4) < rows && m < M && j < R) out[(size_t)m * R + j] = (half_t)(v * drop.scale);
    }
}

// ---- gradient of an adapter matrix --------------------------------------------------------
// out[j, c] = alpha * sum_m P[m, j] * in[m, c] as v_mfma_f32_16x16x32_f16 products whose reduction index is the ROW m:
//   A operand  P^T: lane (j = l % 16, kk = l / 16) holds P[mb + 8*kk .. + 7][j]   (rows j >= R are zero)
//   B operand  in:  lane (cg = l % 16, kk) holds in[mb + 8*kk .. + 7][col]         for ONE column per MFMA
// A lane loads eight 16-byte pieces, rows mb + 8*kk + e (e = 0..7) x columns c0 + 8*cg .. + 7 (256 contiguous bytes
// per 16 lanes and row), and turns the 8 x 8 block around in registers with 32 byte permutes; MFMA i of the eight
// then multiplies column c0 + 8*cg + i.  A wavefront so consumes a block of 32 rows x 128 columns (8 KB) with 8
// loads, 32 permutes and 8 MFMAs per 16 adapter rows; the kernel is bound by its loads.  P for the block (32 x R
// values, R even and at most 32) is fetched with 4-byte loads and transposed through a wavefront-private LDS tile.
// Workgroup = 4 wavefronts on one 128-column strip and `rows_per_wg` rows (wavefront w takes the 32-row blocks
// w, w + 4, ...); the sum over wavefronts goes through LDS, the sum over the gridDim.y workgroups of a strip through
// fp32 partial tiles [split][strip][R][128] that lora_grad_reduce_kernel adds in a fixed order (bit-reproducible).
constexpr int kG2Waves = 4, kG2Cols = 128, kG2PadRows = 40;

// One or two gradients per launch (blockIdx.z): the two adapter gradients of a layer share M, R and alpha and are
// independent, so they go out side by side.  Workgroups beyond a problem's own grid leave at once.
struct GradProb {
    const half_t* P;          // [M, R]
    const half_t* in;         // [M, C]
    float* out;               // through o_sr, o_sc
    float* part;              // partial tiles [splits][col_blocks][R][128]
    int o_sr, o_sc, C, col_blocks, splits, rows_per_wg;
    DropArgs drop;            // dropout mask applied to `in` (thr15 == 0: none); the result carries drop.scale
};
struct GradArgs {
    GradProb p[2];
    float alpha;
    int M;
};


template <int NPL>
struct G2Regs { uint4_t d[8]; uint32_t p[NPL]; };

template <bool DROP, int RB>    // RB = ceil(R / 16) A operands (1 or 2); R is even
__global__ __launch_bounds__(64 * kG2Waves) void lora_grad_kernel(GradArgs ga, int R) {
    const GradProb& q = ga.p[blockIdx.z];
    if ((int)blockIdx.x >= q.col_blocks || (int)blockIdx.y >= q.splits) return;       // uniform over the workgroup
    constexpr int NPL = 4 * RB;                                                       // 4-byte loads of P per lane and block
    __shared__ float red[kG2Waves][16][kG2Cols];                                      // 32 KB
    __shared__ __attribute__((aligned(16))) half_t pt[kG2Waves][16 * RB][kG2PadRows]; // P^T of the current block
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int cg = lane & 15, kk = lane >> 4;
    const int C = q.C, M = ga.M;
    const int row_bytes = C * 2;
    const int c0 = blockIdx.x * kG2Cols + 8 * cg;
    const int m_wg = blockIdx.y * q.rows_per_wg;
    const int m_end = min(m_wg + q.rows_per_wg, M);
    const rsrc_t rs_in = make_rsrc(q.in, (unsigned)m_end * (unsigned)row_bytes);       // rows past m_end read as zero
    const rsrc_t rs_p = make_rsrc(q.P, (unsigned)m_end * (unsigned)(R * 2));
    int voff[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) voff[e] = c0 < C ? (8 * kk + e) * row_bytes + c0 * 2 : kFarOffset;
    // this lane's share of a block of P: the pairs i = lane, lane + 64, ... of the 32 x R block
    // (row i / (R/2), columns 2 * (i % (R/2)) and the next)
    const int hr = R >> 1;
    int pvoff[NPL], pdst[NPL];
#pragma unroll
    for (int t = 0; t < NPL; ++t) {
        const int i = lane + 64 * t, m = i / hr, j = 2 * (i - m * hr);
        pvoff[t] = i < 32 * hr ? i * 4 : kFarOffset;
        pdst[t] = i < 32 * hr ? j * kG2PadRows + m : -1;
    }
    half_t* const ptw = &pt[wave][0][0];
    for (int i = lane; i < 16 * RB * kG2PadRows; i += 64) ptw[i] = (half_t)0.f;   // rows j >= R stay zero
    const DropArgs drop = q.drop;
    const uint32_t thr_pair = drop.thr15 | (drop.thr15 << 16);

    float4_t acc[RB][8];
#pragma unroll
    for (int b = 0; b < RB; ++b)
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[b][i] = float4_t{0.f, 0.f, 0.f, 0.f};

    auto load_block = [&](G2Regs<NPL>& x, int mb) {
        const bool live = mb < m_end;
        const int soff = live ? mb * row_bytes : kFarOffset;
        const int soff_p = live ? mb * R * 2 : kFarOffset;
#pragma unroll
        for (int t = 0; t < NPL; ++t) x.p[t] = buf_load32(rs_p, pvoff[t], soff_p);
#pragma unroll
        for (int e = 0; e < 8; ++e) x.d[e] = buf_load128(rs_in, voff[e], soff);
    };
    auto consume = [&](G2Regs<NPL>& x, int mb) {
        if (DROP && drop.thr15) {                 // uniform: the mask belongs to one problem of a pair
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint32_t key = drop_row_key(drop, (uint32_t)(mb + 8 * kk + e));
                const uint32_t pr = (uint32_t)(c0 >> 1);
                x.d[e].x &= drop_keep_mask(drop_word(drop, key, pr), thr_pair);
                x.d[e].y &= drop_keep_mask(drop_word(drop, key, pr + 1), thr_pair);
                x.d[e].z &= drop_keep_mask(drop_word(drop, key, pr + 2), thr_pair);
                x.d[e].w &= drop_keep_mask(drop_word(drop, key, pr + 3), thr_pair);
            }
        }
#pragma unroll
        for (int t = 0; t < NPL; ++t)
            if (pdst[t] >= 0) {
                ptw[pdst[t]] = __builtin_bit_cast(half_t, (uint16_t)(x.p[t] & 0xFFFFu));
                ptw[pdst[t] + kG2PadRows] = __builtin_bit_cast(half_t, (uint16_t)(x.p[t] >> 16));
            }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        half8_t aop[RB];
#pragma unroll
        for (int b = 0; b < RB; ++b) aop[b] = *reinterpret_cast<const half8_t*>(ptw + (16 * b + cg) * kG2PadRows + 8 * kk);
        __builtin_amdgcn_wave_barrier();
        // 8 x 8 turn: tr[c][q] = (row 2q, row 2q + 1) of column c of this lane's block
        uint32_t tr[8][4];
#pragma unroll
        for (int qq = 0; qq < 4; ++qq) {
            const uint4_t r0 = x.d[2 * qq], r1 = x.d[2 * qq + 1];
            const uint32_t a0[4] = {r0.x, r0.y, r0.z, r0.w}, a1[4] = {r1.x, r1.y, r1.z, r1.w};
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                tr[2 * p][qq] = __builtin_amdgcn_perm(a1[p], a0[p], 0x05040100u);
                tr[2 * p + 1][qq] = __builtin_amdgcn_perm(a1[p], a0[p], 0x07060302u);
            }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint4_t bq = {tr[i][0], tr[i][1], tr[i][2], tr[i][3]};
#pragma unroll
            for (int b = 0; b < RB; ++b)
                acc[b][i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aop[b], __builtin_bit_cast(half8_t, bq), acc[b][i], 0, 0, 0);
        }
    };

    // blocks w, w + 4, ... of the workgroup's rows; the next block's loads are in flight while one is consumed
    const int step = 32 * kG2Waves;
    G2Regs<NPL> xa, xb;
    int mb = m_wg + 32 * wave;
    load_block(xa, mb);
    for (; mb < m_end; mb += 2 * step) {
        load_block(xb, mb + step);
        consume(xa, mb);
        load_block(xa, mb + 2 * step);
        if (mb + step < m_end) consume(xb, mb + step);
    }
    const bool direct = q.splits == 1;
    const float alpha = ga.alpha * drop.scale;
    float* tile = q.part + ((size_t)blockIdx.y * q.col_blocks + blockIdx.x) * (size_t)(R * kG2Cols);
#pragma unroll
    for (int b = 0; b < RB; ++b) {
        if (b > 0) __syncthreads();
        // acc[b][i][r]: adapter row j = 16*b + 4*kk + r, column 8*cg + i of the strip
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float* dst = &red[wave][4 * kk + r][8 * cg];
            *reinterpret_cast<float4_t*>(dst) = float4_t{acc[b][0][r], acc[b][1][r], acc[b][2][r], acc[b][3][r]};
            *reinterpret_cast<float4_t*>(dst + 4) = float4_t{acc[b][4][r], acc[b][5][r], acc[b][6][r], acc[b][7][r]};
        }
        __syncthreads();
        const int nj = min(16, R - 16 * b);
        for (int o = threadIdx.x; o < nj * kG2Cols; o += 64 * kG2Waves) {
            const int jl = o >> 7, cl = o & (kG2Cols - 1), j = 16 * b + jl;
            const float v = (red[0][jl][cl] + red[1][jl][cl]) + (red[2][jl][cl] + red[3][jl][cl]);
            if (direct) {
                const int cc = blockIdx.x * kG2Cols + cl;
                if (cc < C) q.out[(size_t)j * q.o_sr + (size_t)cc * q.o_sc] = alpha * v;
            } else {
                tile[j * kG2Cols + cl] = v;
            }
        }
    }
}

// Adds the `splits` partial tiles of every strip in order and writes the scaled result through the caller's strides.
__global__ __launch_bounds__(256) void lora_grad_reduce_kernel(GradArgs ga, int R) {
    const GradProb& q = ga.p[blockIdx.y];
    const int total = q.col_blocks * R * kG2Cols;              // one split's tiles: [strip][j][column]
    const int t = blockIdx.x * 256 + threadIdx.x;
    if (q.splits <= 1 || t >= total) return;                   // a single split was written directly
    const float* __restrict__ part = q.part;
    float v = 0.f;
    int s = 0;
    for (; s + 8 <= q.splits; s += 8) {
        float u[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) u[i] = part[(size_t)(s + i) * total + t];
#pragma unroll
        for (int i = 0; i < 8; ++i) v += u[i];
    }
    for (; s < q.splits; ++s) v += part[(size_t)s * total + t];
    const int bx = t / (R * kG2Cols), o = t - bx * (R * kG2Cols);
    const int j = o >> 7, cc = bx * kG2Cols + (o & (kG2Cols - 1));
    if (cc < q.C) q.out[(size_t)j * q.o_sr + (size_t)cc * q.o_sc] = ga.alpha * q.drop.scale * v;
}

// keep[m, c] = 1 where dropout keeps element (m, c), else 0: the mask the kernels above regenerate, written out
// for callers (and tests) that need to see it.
__global__ __launch_bounds__(256) void dropout_keep_kernel(uint8_t* __restrict__ keep, int M, int C, DropArgs drop) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;              // one column pair per thread
    const long pairs = (long)M * (C / 2);
    if (i >= pairs) return;
    const int m = (int)(i / (C / 2)), pr = (int)(i - (long)m * (C / 2));
    const uint32_t w = drop_word(drop, drop_row_key(drop, (uint32_t)m), (uint32_t)pr);
    keep[(size_t)m * C + 2 * pr] = (w & 0x7FFFu) >= drop.thr15;
    keep[(size_t)m * C + 2 * pr + 1] = ((w >> 16) & 0x7FFFu) >= drop.thr15;
}

// 128-column strips; enough row splits for about two workgroups per CU over both problems of a pair (their partial
// tiles cost 2 * splits * R * C * 4 bytes of traffic); rows per workgroup a multiple of 128 (4 wavefronts x 32 rows).
struct GradPlan { int col_blocks, splits, rows_per_wg; };
inline GradPlan plan_grad(int M, int C) {
    GradPlan g;
    g.col_blocks = (C + kG2Cols - 1) / kG2Cols;
    int splits = (384 + g.col_blocks - 1) / g.col_blocks;
    if (splits > 64) splits = 64;
    if (splits < 1) splits = 1;
    const int unit = 32 * kG2Waves;
    g.rows_per_wg = ((M + splits - 1) / splits + unit - 1) / unit * unit;
    g.splits = (M + g.rows_per_wg - 1) / g.rows_per_wg;
    return g;
}

}  // namespace q4

template <int RB, int WL, bool F32, int RQ>
static void launch_down_kernel(const q4::half_t* ip, const void* w, int w_sr, int w_sc, q4::half_t* op,
                               int M, int C, int R, const q4::DropArgs& drop, hipStream_t stream) {
    // rows of `in` per workgroup: 16 fill the MFMA operand, but with few rows that leaves compute units idle and
    // the kernel is bound by the latency of its single burst of loads, so smaller blocks spread it out
    int rows = 16;
    while (rows > 4 && (M + rows - 1) / rows < 256) rows >>= 1;
    hipLaunchKernelGGL((q4::lora_down_kernel<RB, WL, F32, RQ>), dim3((M + rows - 1) / rows), dim3(64 * q4::kDownWaves), 0,
                       stream, ip, w, w_sr, w_sc, op, M, C, R, rows, drop);
}

template <int WL, bool F32>
static void launch_down_rb(const q4::half_t* ip, const void* w, int w_sr, int w_sc, q4::half_t* op,
                           int M, int C, int R, const q4::DropArgs& drop, hipStream_t stream) {
    switch ((R + 15) / 16) {
        case 1: launch_down_kernel<1, WL, F32, 0>(ip, w, w_sr, w_sc, op, M, C, R, drop, stream); break;
        case 2: launch_down_kernel<2, WL, F32, 0>(ip, w, w_sr, w_sc, op, M, C, R, drop, stream); break;
        case 3: launch_down_kernel<3, WL, F32, 0>(ip, w, w_sr, w_sc, op, M, C, R, drop, stream); break;
        default: launch_down_kernel<4, WL, F32, 0>(ip, w, w_sr, w_sc, op, M, C, R, drop, stream); break;
    }
}

template <int WL, bool F32>
static void launch_down_staged(const q4::half_t* ip, const void* w, int w_sr, int w_sc, q4::half_t* op,
                             int M, int C, int R, const q4::DropArgs& drop, hipStream_t stream) {
    switch ((R + 3) / 4) {
        case 1: launch_down_kernel<1, WL, F32, 1>(ip, w, w_sr, w_sc, op, M, C, R, drop, stream); break;
        case 2: launch_down_kernel<1, WL, F32, 2>(ip, w, w_sr, w_sc, op, M, C, R, drop, stream); break;
        case 3: launch_down_kernel<1, WL, F32, 3>(ip, w, w_sr, w_sc, op, M, C, R, drop, stream); break;
        default: launch_down_kernel<1, WL, F32, 4>(ip, w, w_sr, w_sc, op, M, C, R, drop, stream); break;
    }
}

extern "C" int q4_launch_lora_down(const void* in, const void* w, int w_sr, int w_sc, int w_is_f32, void* out,
                                   int M, int C, int R, const q4::DropArgs* dropp, hipStream_t stream) {
    using namespace q4;
    const DropArgs drop = dropp ? *dropp : DropArgs{0u, 0u, 0u, 1.0f};
    const half_t* ip = reinterpret_cast<const half_t*>(in);
    half_t* op = reinterpret_cast<half_t*>(out);
    const bool base16 = (reinterpret_cast<uintptr_t>(w) & 15u) == 0;
    const int vec = w_is_f32 ? 4 : 8;                       // elements per 16 bytes
    if (w_sc == 1 && base16 && w_sr % 4 == 0 && R <= 16) {
        if (w_is_f32) launch_down_staged<kRowsT, true>(ip, w, w_sr, w_sc, op, M, C, R, drop, stream);
        else launch_down_staged<kRowsT, false>(ip, w, w_sr, w_sc, op, M, C, R, drop, stream);
    } else if (w_sc == 1 && base16 && w_sr % vec == 0) {
        if (w_is_f32) launch_down_rb<kRows, true>(ip, w, w_sr, w_sc, op, M, C, R, drop, stream);
        else launch_down_rb<kRows, false>(ip, w, w_sr, w_sc, op, M, C, R, drop, stream);
    } else if (w_sr == 1 && base16 && w_sc % 4 == 0 && R % 4 == 0 && R <= 16 && w_sc >= R) {
        if (w_is_f32) launch_down_staged<kCols, true>(ip, w, w_sr, w_sc, op, M, C, R, drop, stream);
        else launch_down_staged<kCols, false>(ip, w, w_sr, w_sc, op, M, C, R, drop, stream);
    } else {
        if (w_is_f32) launch_down_rb<kAny, true>(ip, w, w_sr, w_sc, op, M, C, R, drop, stream);
        else launch_down_rb<kAny, false>(ip, w, w_sr, w_sc, op, M, C, R, drop, stream);
    }
    return hipGetLastError() == hipSuccess ? 0 : -4;
}

extern "C" size_t q4_lora_grad_workspace(int M, int C, int R) {
    const q4::GradPlan g = q4::plan_grad(M, C);
    return g.splits == 1 ? 0 : (size_t)g.splits * g.col_blocks * R * q4::kG2Cols * sizeof(float);
}

static q4::GradProb make_grad_prob(const void* P, const void* in, float* out, int o_sr, int o_sc, int M, int C, int R,
                                   float* part, const q4::DropArgs* drop = nullptr) {
    const q4::GradPlan g = q4::plan_grad(M, C);
    q4::GradProb q;
    q.P = reinterpret_cast<const q4::half_t*>(P);
    q.in = reinterpret_cast<const q4::half_t*>(in);
    q.out = out;
    q.part = part;
    q.o_sr = o_sr; q.o_sc = o_sc; q.C = C;
    q.col_blocks = g.col_blocks; q.splits = g.splits; q.rows_per_wg = g.rows_per_wg;
    q.drop = drop ? *drop : q4::DropArgs{0u, 0u, 0u, 1.0f};
    return q;
}

static int launch_grad(const q4::GradArgs& ga, int nprob, int R, hipStream_t stream) {
    using namespace q4;
    int gx = 0, gy = 0, rx = 0;
    bool any_split = false, any_drop = false;
    for (int i = 0; i < nprob; ++i) {
        gx = ga.p[i].col_blocks > gx ? ga.p[i].col_blocks : gx;
        gy = ga.p[i].splits > gy ? ga.p[i].splits : gy;
        const int rb = (ga.p[i].col_blocks * R * kG2Cols + 255) / 256;
        rx = rb > rx ? rb : rx;
        any_split = any_split || ga.p[i].splits > 1;
        any_drop = any_drop || ga.p[i].drop.thr15 != 0;
    }
    const dim3 grid(gx, gy, nprob), block(64 * kG2Waves);
    if (R <= 16) {
        if (any_drop) hipLaunchKernelGGL((lora_grad_kernel<true, 1>), grid, block, 0, stream, ga, R);
        else hipLaunchKernelGGL((lora_grad_kernel<false, 1>), grid, block, 0, stream, ga, R);
    } else {
        if (any_drop) hipLaunchKernelGGL((lora_grad_kernel<true, 2>), grid, block, 0, stream, ga, R);
        else hipLaunchKernelGGL((lora_grad_kernel<false, 2>), grid, block, 0, stream, ga, R);
    }
    if (any_split) hipLaunchKernelGGL(lora_grad_reduce_kernel, dim3(rx, nprob), dim3(256), 0, stream, ga, R);
    return hipGetLastError() == hipSuccess ? 0 : -4;
}

extern "C" int q4_launch_lora_grad(const void* P, const void* in, float* out, int o_sr, int o_sc, float alpha,
                                   int M, int C, int R, const q4::DropArgs* drop, void* workspace, hipStream_t stream) {
    q4::GradArgs ga;
    ga.p[0] = make_grad_prob(P, in, out, o_sr, o_sc, M, C, R, reinterpret_cast<float*>(workspace), drop);
    ga.p[1] = ga.p[0];
    ga.alpha = alpha;
    ga.M = M;
    return launch_grad(ga, 1, R, stream);
}

extern "C" int q4_launch_dropout_keep(uint8_t* keep, int M, int C, const q4::DropArgs* drop, hipStream_t stream) {
    const long pairs = (long)M * (C / 2);
    hipLaunchKernelGGL(q4::dropout_keep_kernel, dim3((unsigned)((pairs + 255) / 256)), dim3(256), 0, stream, keep, M, C, *drop);
    return hipGetLastError() == hipSuccess ? 0 : -4;
}

// Two gradients with the same M, R and alpha in one launch (plus one launch for both reductions); the workspace
// holds the partial tiles of the first problem followed by those of the second.
extern "C" int q4_launch_lora_grad_pair(const void* P1, const void* in1, float* out1, int o1_sr, int o1_sc, int C1,
                                        const void* P2, const void* in2, float* out2, int o2_sr, int o2_sc, int C2,
                                        float alpha, int M, int R, const q4::DropArgs* drop1, void* workspace,
                                        hipStream_t stream) {
    q4::GradArgs ga;
    float* ws = reinterpret_cast<float*>(workspace);
    ga.p[0] = make_grad_prob(P1, in1, out1, o1_sr, o1_sc, M, C1, R, ws, drop1);      // the mask applies to in1 only
    ga.p[1] = make_grad_prob(P2, in2, out2, o2_sr, o2_sc, M, C2, R,
                             ws ? ws + q4_lora_grad_workspace(M, C1, R) / sizeof(float) : nullptr);
    ga.alpha = alpha;
    ga.M = M;
    return launch_grad(ga, 2, R, stream);
}
