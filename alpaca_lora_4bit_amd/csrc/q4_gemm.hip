// Fused dequantize + fp16 MFMA GEMMs (MFMA-bound):
//   forward   y [M,N] = x  [M,K] @ W      (+ bias) (+ xa  [M,R] @ lora_bt [R,N])
//   backward  dx[M,K] = dy [M,N] @ W^T             (+ dyb [M,R] @ lora_a  [R,K])
// W is never materialised in HBM: each workgroup dequantizes the [64 x 128] slab of W its
// current step needs straight into LDS, with the reference's three fp16 roundings
// (src/alpaca_lora_4bit/quant_cuda/quant_cuda_kernel.cu:1146-1151), so the product equals
// torch.matmul(x, recons(W)) of matmul_utils_4bit.py:122-126 up to fp32 summation order.
//
// Tiling.  A workgroup computes a BM x 128 output tile with 2*WGM wavefronts (WGM along M, 2
// along N), each owning (BM/WGM) x 64 outputs as (BM/WGM/32) x 2 accumulators of
// v_mfma_f32_32x32x16_f16.  From 129 rows on BM = 256 with 8 wavefronts of 64 x 64 (two per SIMD:
// while one waits or dequantizes the other multiplies, and one dequantized slab of W serves 256
// activation rows), with the reduction split over several workgroups when there are too few tiles
// for the CUs (plan_gemm); fewer rows use BM = 128 with 4 wavefronts.  The reduction runs in steps
// of 64.  Both LDS tiles are stored "row = output index, minor = reduction index" with 8 halves of
// padding per row (stride 144 B): the 128-bit operand fetches of 16 consecutive lanes then hit
// 64 distinct banks.  LDS is double buffered in four distinct arrays (110 KB at BM = 256).
//
// Pipeline (hand-scheduled; with one or two wavefronts per SIMD little else hides a stall):
//   * global loads of stage s+2 go to a second register set through buffer instructions whose
//     per-thread offsets are computed once (zero address arithmetic in the loop; rows beyond M
//     fall outside the buffer descriptor and read as zero);
//   * the registers of stage s+1 are dequantized into the other LDS buffer in 16 small slices;
//   * each of the 16 MFMAs of stage s is followed by one such slice / load batch / LDS
//     store and a scheduling barrier that pins the interleaving, since an MFMA keeps the matrix
//     pipe busy for 8 passes during which the wavefront may issue other instructions;
//   * the workgroup barrier sits a few MFMAs before the end of the step and the first operand
//     fragments of stage s+1 are fetched right after it, under the remaining MFMAs.
//
// The LoRA term is one more reduction step whose A operand is the precomputed [M,R] rank-R
// activation and whose B operand is the fp16 adapter matrix: no second pass over the output.
// The epilogue transposes the accumulators through LDS so that y is written in 16-byte pieces.
#include "q4_common.hpp"
#include <stdlib.h>
#include <type_traits>

namespace q4 {

constexpr int BN = 128, BK = 64;
constexpr int LDS_STRIDE = BK + 8;   // halves

struct GemmArgs {
    const half_t* a;          // fwd: x [M,K]      bwd: dy [M,N]
    const uint32_t* qweight;  // [K/8, N]
    const uint32_t* qzeros;   // [G, N/8]
    const half_t* scales;     // [G, N]
    const int32_t* g_idx;     // [K] or null
    int groupsize;
    uint32_t gs_inv31;        // ceil(2^31 / (groupsize / 64)): reduction offset -> group without a division
    const half_t* bias;       // fwd only, [N] or null
    const half_t* la;         // fwd: xa [M,R]     bwd: dyb [M,R]   (or null)
    const void* lb;           // adapter matrix (fp16 or fp32), element (r, c) at lb[r*lb_sr + c*lb_sc]; fwd: c = n, bwd: c = k
    int lb_sr, lb_sc, lb_is_f32;
    float lb_scale;           // multiplied into the adapter matrix when it is staged in LDS
    int R;
    half_t* out;              // fwd: y [M,N]      bwd: dx [M,K]
    int M, K, N, G;
    int phase_step;           // bits 0-7: rotation of the reduction loop per row tile, in steps of 64; bits 8+: row tiles per group of the tile order
    float* part;              // split-K: fp32 partial outputs [gridDim.z][M][part_cols] (gridDim.z > 1 only)
    int col_tile0;            // first column tile of this launch (a launch may cover a range of column tiles)
    int part_cols;            // columns held by `part`: those of this launch's column tiles
    DropArgs drop;            // thr15 != 0: the adapter term of out[m, c] is kept only where dropout keeps (m, c)
};

// Which output tile a workgroup computes, and where in the reduction it starts.
//  * Workgroups are handed to the 8 XCDs round-robin in dispatch order.  The ids are permuted so that one
//    XCD owns a contiguous range of tiles, ordered in groups of `rg` row tiles: all column tiles of a group,
//    then the next group.  The 32 workgroups an XCD runs at a time then share 2 slabs of activations and 16
//    column tiles of W (about 4 MB each at K = 4096, what its L2 holds) instead of every row tile of a few
//    columns: with many row tiles the activations would otherwise stream from HBM once per column tile
//    (8192 x 4096 x 4096: 306 -> 260 us; no shape slower).
//  * Activation rows of a power-of-two pitch (K = 4096: 8 KB) put one reduction slab of ALL rows into
//    a single L2 channel; workgroups marching through the reduction in lockstep then queue on that one
//    channel.  Row tile r therefore starts its (cyclic) reduction loop phase_step * r steps later.
struct TileMap {
    int tile_c, tile_r, phase;
};
__device__ __forceinline__ TileMap map_tile(int phase_step, int nsteps, int col_tile0) {   // nsteps: steps of THIS workgroup
    const int nc = gridDim.x, nr = gridDim.y, total = nc * nr;
    int id = blockIdx.y * nc + blockIdx.x;
    if (total % 8 == 0) id = (id % 8) * (total / 8) + id / 8;
    TileMap m;
    const int rg = phase_step >> 8;                   // row tiles per group (0: column-major over all row tiles)
    phase_step &= 0xff;
    const int grouped = rg > 0 ? (nr / rg) * rg * nc : 0;
    if (id < grouped) {
        // groups of rg row tiles: all column tiles of a group, then the next group
        const int gi = id / (rg * nc), rem = id - gi * rg * nc;
        m.tile_c = rem / rg;
        m.tile_r = gi * rg + (rem - m.tile_c * rg);
    } else {
        const int left = rg > 0 ? nr % rg : nr, base = nr - left, rem = id - grouped;
        m.tile_c = rem / left;
        m.tile_r = base + (rem - m.tile_c * left);
    }
    m.tile_c += col_tile0;
    m.phase = (m.tile_r * phase_step) % nsteps;
    return m;
}
// Split-K: gridDim.z workgroups share an output tile; workgroup z owns `cnt` consecutive steps from `begin`.
struct StepRange {
    int begin, cnt;
};
__device__ __forceinline__ StepRange split_steps(int nsteps, int z, int S) {
    const int base = nsteps / S, rem = nsteps - base * S;
    StepRange r;
    r.cnt = base + (z < rem ? 1 : 0);
    r.begin = z * base + min(z, rem);
    return r;
}
// reduction offset of pipeline stage `stage` (stages past the end repeat the last one: harmless reloads)
__device__ __forceinline__ int red_of(int stage, StepRange sr, int phase) {
    int v = min(stage, sr.cnt - 1) + phase;
    if (v >= sr.cnt) v -= sr.cnt;
    return (sr.begin + v) * BK;
}

// Group of reduction row k (a multiple of 64; sequential groups of a multiple of 64 rows):
// floor((k/64) / (groupsize/64)) as a multiply-high, exact while k * groupsize < 2^40.
__device__ __forceinline__ int group_of(const GemmArgs& a, int k) {
    return (int)__umulhi((uint32_t)k >> 5, a.gs_inv31);
}

__device__ __forceinline__ float adapter_at(const GemmArgs& a, size_t idx) {
    return a.lb_is_f32 ? reinterpret_cast<const float*>(a.lb)[idx] : (float)reinterpret_cast<const half_t*>(a.lb)[idx];
}
// rn16(rn16(s*q) - zero) for a pair of codes given as (0x6400 | q): one fused multiply-add
// computes s*(1024+q) - 1024*s = s*q with a single rounding (1024*s is exact), i.e. exactly
// rn16(s*q); the subtraction of the zero term is the third rounding.  Needs |s| < 64 so that
// 1024*s does not overflow (checked on the host; larger scales take the unfused path).
__device__ __forceinline__ half2_t dequant_pair_magic(uint32_t codes_or_magic, half2_t s, half2_t s1024, half2_t zero) {
    const half2_t p = __builtin_elementwise_fma(as_half2(codes_or_magic), s, -s1024);
    return p - zero;
}

template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

struct SlabRsrc {
    rsrc_t w, s, z;
};

// ---- weight slab loaders: global -> registers -> (dequant) -> LDS ----------------------
// The dequantization of a slab is cut into kSlices = 16 pieces so that the main loop can hand
// the vector ALU one piece between two MFMAs.  With GIDX (act-order, or scales too large for
// the fused form) rows gather (scale, zero) through g_idx and everything happens in piece 0.
//
// Forward: slab = 64 rows (k) x 128 columns (n); LDS row = column n, minor = k.
// A thread owns ONE column for the whole kernel and 4 packed words (32 rows) per step;
// piece I handles pair I%4 of word I/4 and the word goes to LDS with its last piece.
template <bool GIDX, int NT, int BNT = 128>
struct FwdSlab {
    static constexpr int NW = 8 * BNT / NT;       // packed words per thread per step (4 or 2)
    static constexpr int WSTEP = NT / BNT;        // word-row distance between a thread's words
    static constexpr int kSlices = 4 * NW;
    uint32_t w[NW];
    uint32_t s_raw;  // fp16 bits of the scale of (current group, own column); decoded in the slices
    uint32_t z_raw;  // packed zero word holding the own column's code
    uint32_t o[4];
    int col, wr0;    // column 0..127 of the tile; first word-row within the slab, then +WSTEP per word
    int voff_w, voff_s, voff_z, wstride;
    __device__ __forceinline__ void init(int t, const GemmArgs& a, int n0) {
        col = t % BNT; wr0 = t / BNT;
        wstride = WSTEP * a.N * 4;
        voff_w = (wr0 * a.N + n0 + col) * 4;
        voff_s = (n0 + col) * 2;
        voff_z = ((n0 + col) >> 3) * 4;
    }
    // raw loads only: any arithmetic on the loaded values here would wait for them before the MFMAs.
    // The loads of a slab are kLoads separate pieces so that the main loop can issue them one at a time.
    static constexpr int kLoads = GIDX ? NW : NW + 2;
    template <int I>
    __device__ __forceinline__ void load_part(const GemmArgs& a, const SlabRsrc& r, int kred0) {
        if constexpr (I < NW) {
            w[I] = buf_load32(r.w, voff_w + I * wstride, (kred0 >> 3) * a.N * 4);
        } else if constexpr (I == NW) {
            s_raw = buf_load16(r.s, voff_s, group_of(a, kred0) * a.N * 2);
        } else {
            z_raw = buf_load32(r.z, voff_z, group_of(a, kred0) * (a.N >> 3) * 4);
        }
    }
    __device__ __forceinline__ void load(const GemmArgs& a, const SlabRsrc& r, int, int kred0) {
        static_for<0, kLoads>([&](auto ic) { load_part<decltype(ic)::value>(a, r, kred0); });
    }
    // what the slices of a step need of (scale, zero) of the step's group, computed once per group change
    struct Prep { half2_t s2, zero2, s1024; };
    __device__ __forceinline__ Prep make_prep(int n0) const {
        Prep pr;
        pr.s2 = as_half2(s_raw | (s_raw << 16));
        const uint32_t z_cur = (z_raw >> (((n0 + col) & 7) * 4)) & 0xFu;
        pr.zero2 = zero_term(pr.s2, z_cur, z_cur);
        pr.s1024 = pr.s2 * half2_t{(half_t)1024.f, (half_t)1024.f};
        return pr;
    }
    template <int I>
    __device__ __forceinline__ void store_slice(const GemmArgs& a, int n0, int kred0, half_t* sB, const Prep& pr) {
        const int n = n0 + col;
        if constexpr (GIDX) {
            if constexpr (I == 0) {
                const int ncol8 = a.N >> 3;
                const int zsh = (n & 7) * 4;
                const half2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f};
#pragma unroll
                for (int i = 0; i < NW; ++i) {
                    const int wr = wr0 + WSTEP * i;
                    const uint32_t lo = w[i] & 0x0F0F0F0Fu, hi = (w[i] >> 4) & 0x0F0F0F0Fu;
                    uint32_t oo[4];
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        const uint32_t codes = __builtin_amdgcn_perm(hi, lo, 0x0c040c00u + 0x00010001u * p) | kMagic;
                        const int k = kred0 + 8 * wr + 2 * p;
                        const int g0 = a.g_idx[k], g1 = a.g_idx[k + 1];
                        const half2_t s2 = {a.scales[(size_t)g0 * a.N + n], a.scales[(size_t)g1 * a.N + n]};
                        const half2_t zero2 = zero_term(s2, (a.qzeros[(size_t)g0 * ncol8 + (n >> 3)] >> zsh) & 0xFu,
                                                        (a.qzeros[(size_t)g1 * ncol8 + (n >> 3)] >> zsh) & 0xFu);
                        oo[p] = as_u32(dequant_pair(as_half2(codes) - k1024, s2, zero2));
                    }
                    *reinterpret_cast<uint4_t*>(sB + col * LDS_STRIDE + 8 * wr) = uint4_t{oo[0], oo[1], oo[2], oo[3]};
                }
            }
        } else {
            constexpr int i = I / 4, p = I % 4;
            const uint32_t lo = w[i] & 0x0F0F0F0Fu;          // bytes e0 e2 e4 e6
            const uint32_t hi = (w[i] >> 4) & 0x0F0F0F0Fu;   // bytes e1 e3 e5 e7
            const uint32_t codes = __builtin_amdgcn_perm(hi, lo, 0x0c040c00u + 0x00010001u * p) | kMagic;
            o[p] = as_u32(dequant_pair_magic(codes, pr.s2, pr.s1024, pr.zero2));
            if constexpr (p == 3)
                *reinterpret_cast<uint4_t*>(sB + col * LDS_STRIDE + 8 * (wr0 + WSTEP * i)) = uint4_t{o[0], o[1], o[2], o[3]};
        }
    }
    __device__ __forceinline__ void fetch_tab(const unsigned char*, int) {}
    // LoRA step: B operand = adapter matrix [R, N]; LDS row = column n, minor = r (zero padded to 64).
    __device__ __forceinline__ void store_lora(const GemmArgs& a, int n0, half_t* sB, int t) const {
        for (int idx = t; idx < BNT * BK; idx += NT) {
            const int r = idx / BNT, c = idx % BNT;
            sB[c * LDS_STRIDE + r] = (r < a.R) ? (half_t)(a.lb_scale * adapter_at(a, (size_t)r * a.lb_sr + (size_t)(n0 + c) * a.lb_sc))
                                               : (half_t)0.f;
        }
    }
};

// Backward: output columns are rows k of W, the reduction runs over n.
// Slab = 128 rows (k) x 64 columns (n); LDS row = k, minor = n.
// A thread owns one word-row (8 output rows) and 4 adjacent columns per step (one 128-bit load).
// With 512 threads two threads share a load and split the word-row's 8 rows 4 + 4.
// Piece I dequantizes columns (0,1) [I even] or (2,3) [I odd] of the thread's row I/2; the
// 8-byte row segment goes to LDS with the odd piece.
// TAB: the scales and the zero terms rn16(s * (z + 1)) of the tile's group sit in an LDS table for every column n,
// per column pair as (s_a, s_b, zero_a, zero_b) (filled once per workgroup), and come from there: one 16-byte LDS
// read per step instead of two more global loads and the zero-term arithmetic of every step.
template <bool GIDX, int NT, bool TAB = false, int BNT = 128>
struct BwdSlab {
    static constexpr int RPT = 16 * BNT / NT;     // rows of the word-row handled by one thread (8 or 4)
    static constexpr int kSlices = 2 * RPT;
    uint4_t w;
    uint2_t sv;
    uint32_t zw, o01;
    uint4_t tv;                                   // TAB: (s01, zero01, s23, zero23) of this thread's four columns
    int wr, n4, e0;
    int voff_w, voff_s, voff_z;
    __device__ __forceinline__ void init(int t, const GemmArgs& a, int kout0) {
        wr = (t % (2 * BNT)) >> 4; n4 = t & 15; e0 = (t / (2 * BNT)) * RPT;
        const int g = GIDX ? 0 : (kout0 + 8 * wr) / a.groupsize;      // fixed for the whole kernel
        voff_w = (((kout0 >> 3) + wr) * a.N + 4 * n4) * 4;
        voff_s = (g * a.N + 4 * n4) * 2;
        voff_z = (g * (a.N >> 3) + (n4 >> 1)) * 4;
    }
    static constexpr int kLoads = (GIDX || TAB) ? 1 : 3;
    __device__ __forceinline__ void fetch_tab(const unsigned char* tab, int nred0) {
        tv = *reinterpret_cast<const uint4_t*>(tab + (nred0 + 4 * n4) * 4);
    }
    struct Prep {};
    __device__ __forceinline__ Prep make_prep(int) const { return Prep{}; }
    template <int I>
    __device__ __forceinline__ void load_part(const GemmArgs&, const SlabRsrc& r, int nred0) {
        if constexpr (I == 0) w = buf_load128(r.w, voff_w, nred0 * 4);
        else if constexpr (I == 1) sv = buf_load64(r.s, voff_s, nred0 * 2);
        else zw = buf_load32(r.z, voff_z, (nred0 >> 3) * 4);     // shifted in the slices: no ALU on loaded data here
    }
    __device__ __forceinline__ void load(const GemmArgs& a, const SlabRsrc& r, int, int nred0) {
        static_for<0, kLoads>([&](auto ic) { load_part<decltype(ic)::value>(a, r, nred0); });
    }
    template <int I>
    __device__ __forceinline__ void store_slice(const GemmArgs& a, int kout0, int nred0, half_t* sB, const Prep&) {
        const int n = nred0 + 4 * n4;
        const int zsh = (n4 & 1) * 16;
        const half2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f};
        if constexpr (GIDX) {
            if constexpr (I == 0) {
                const int ncol8 = a.N >> 3;
                const int kbase = kout0 + 8 * wr;
                const uint32_t wj[4] = {w.x, w.y, w.z, w.w};
                uint32_t lo[4], hi[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) { lo[j] = wj[j] & 0x0F0F0F0Fu; hi[j] = (wj[j] >> 4) & 0x0F0F0F0Fu; }
#pragma unroll
                for (int ee = 0; ee < RPT; ++ee) {
                    const int e = e0 + ee;
                    const int g = a.g_idx[kbase + e];
                    const uint2_t s4 = *reinterpret_cast<const uint2_t*>(a.scales + (size_t)g * a.N + n);
                    const uint32_t z4 = a.qzeros[(size_t)g * ncol8 + (n >> 3)] >> zsh;
                    const half2_t s01 = as_half2(s4.x), s23 = as_half2(s4.y);
                    const half2_t z01 = zero_term(s01, z4 & 0xFu, (z4 >> 4) & 0xFu);
                    const half2_t z23 = zero_term(s23, (z4 >> 8) & 0xFu, (z4 >> 12) & 0xFu);
                    const int b = e >> 1;
                    const uint32_t sel = 0x0c000c00u | ((4u + b) << 16) | (uint32_t)b;
                    const uint32_t c01 = ((e & 1) ? __builtin_amdgcn_perm(hi[1], hi[0], sel) : __builtin_amdgcn_perm(lo[1], lo[0], sel)) | kMagic;
                    const uint32_t c23 = ((e & 1) ? __builtin_amdgcn_perm(hi[3], hi[2], sel) : __builtin_amdgcn_perm(lo[3], lo[2], sel)) | kMagic;
                    const uint2_t oo = {as_u32(dequant_pair(as_half2(c01) - k1024, s01, z01)),
                                        as_u32(dequant_pair(as_half2(c23) - k1024, s23, z23))};
                    *reinterpret_cast<uint2_t*>(sB + (8 * wr + e) * LDS_STRIDE + 4 * n4) = oo;
                }
            }
        } else {
            // row e = e0 + I/2 with e0 in {0, 4}: odd/even nibble and byte-in-half are compile-time,
            // the half of the word (e0) is a per-thread shift by 0 or 16 bits
            constexpr int el = I / 2, h = I % 2, b = el >> 1;
            constexpr uint32_t sel = 0x0c000c00u | ((4u + b) << 16) | (uint32_t)b;
            const int e = e0 + el;
            const uint32_t z4 = zw >> zsh;
            const uint32_t wa = (h ? w.z : w.x) >> (4 * e0), wb = (h ? w.w : w.y) >> (4 * e0);   // the two columns of this piece
            const uint32_t na = (el & 1) ? ((wa >> 4) & 0x0F0F0F0Fu) : (wa & 0x0F0F0F0Fu);
            const uint32_t nb = (el & 1) ? ((wb >> 4) & 0x0F0F0F0Fu) : (wb & 0x0F0F0F0Fu);
            const uint32_t codes = __builtin_amdgcn_perm(nb, na, sel) | kMagic;  // (code of column a, of column b) of row e
            half2_t s2, zero2;
            if constexpr (TAB) {
                s2 = as_half2(h ? tv.z : tv.x);
                zero2 = as_half2(h ? tv.w : tv.y);
            } else {
                s2 = as_half2(h ? sv.y : sv.x);
                zero2 = zero_term(s2, (z4 >> (8 * h)) & 0xFu, (z4 >> (8 * h + 4)) & 0xFu);
            }
            const uint32_t r = as_u32(dequant_pair_magic(codes, s2, s2 * k1024, zero2));
            if constexpr (h == 0) o01 = r;
            else *reinterpret_cast<uint2_t*>(sB + (8 * wr + e) * LDS_STRIDE + 4 * n4) = uint2_t{o01, r};
        }
    }
    // LoRA step: B operand = adapter matrix [R, K]; LDS row = k, minor = r.
    __device__ __forceinline__ void store_lora(const GemmArgs& a, int kout0, half_t* sB, int t) const {
        for (int idx = t; idx < BNT * BK; idx += NT) {
            const int r = idx / BNT, c = idx % BNT;
            sB[c * LDS_STRIDE + r] = (r < a.R) ? (half_t)(a.lb_scale * adapter_at(a, (size_t)r * a.lb_sr + (size_t)(kout0 + c) * a.lb_sc))
                                               : (half_t)0.f;
        }
    }
};

// WGM = wavefronts along M (2 or 4); the workgroup has 2*WGM wavefronts = NT threads.
// SZ: how the sequential-group kernels get scale and zero (fewer vector-memory and vector-ALU instructions in the
// main loop; 1.5-2.5 % of the kernel):
//   0  loaded with every step (any group size, any split)
//   1  forward: loaded with the even steps only; needs groups of a multiple of 128 rows and a step order in which
//      steps 2i and 2i+1 of a workgroup lie in one group (host: even split starts, lengths and rotation)
//   2  backward: from an LDS table of the tile's group, filled once (needs the 128 output rows of a tile in one
//      group and room for 4 bytes per column n in dynamic LDS)
// WGN: wavefronts along N (2 or 4), each 64 columns wide: the tile is BM x 64*WGN.
// The body of the kernels below.  `tm`: the output tile; `sr`: this workgroup's share of the reduction; `zsplit` of
// `nsplit`: which share that is (share 0 carries bias and adapter term); `zpart`: index of its fp32 partial tile.
template <int BM, int WGM, bool FWD, bool GIDX, int SZ, int WGN>
__device__ __forceinline__ void gemm_body(const GemmArgs& a, const TileMap tm, const StepRange sr, const int zsplit,
                                          const int nsplit, const int zpart) {
    constexpr int BNT = 64 * WGN;                     // columns of the tile
    static_assert(SZ == 0 || (!GIDX && ((FWD && SZ == 1) || (!FWD && SZ == 2))), "unsupported scale/zero mode");
    extern __shared__ __attribute__((aligned(16))) unsigned char sz_tab[];
    // four distinct LDS objects (not one carved-up array): the compiler can then prove that the
    // writes into one buffer do not alias the reads of the other and is free to interleave them
    __shared__ __attribute__((aligned(16))) half_t sA0[BM * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) half_t sA1[BM * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) half_t sB0[BNT * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) half_t sB1[BNT * LDS_STRIDE];
    constexpr int NT = 64 * WGM * WGN;                // threads per workgroup
    constexpr int WROWS = BM / WGM;                   // output rows per wavefront
    constexpr int TM = WROWS / 32;                    // 32-row accumulator tiles per wavefront
    constexpr int NA = BM * 8 / NT;                   // 16-byte activation loads per thread per step
    constexpr int APASS = NT / 8;                     // activation rows covered by one pass of the workgroup
    constexpr int KS = BK / 16;                       // MFMA reduction sub-steps per step

    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    const int NOUT = FWD ? a.N : a.K;
    const int RED = FWD ? a.K : a.N;
    const int m0 = tm.tile_r * BM;
    const int c0 = tm.tile_c * BNT;          // first output column of the tile
    const int rows_valid = min(BM, a.M - m0);

    // buffer descriptors: activations of this workgroup's rows (rows beyond M read as zero), weights
    const rsrc_t rs_a = make_rsrc(a.a + (size_t)m0 * RED, (unsigned)rows_valid * (unsigned)RED * 2u);
    SlabRsrc rs;
    rs.w = make_rsrc(a.qweight, (unsigned)(a.K >> 3) * (unsigned)a.N * 4u);
    rs.s = make_rsrc(a.scales, (unsigned)a.G * (unsigned)a.N * 2u);
    rs.z = make_rsrc(a.qzeros, (unsigned)a.G * (unsigned)(a.N >> 3) * 4u);

    // activation tile: BM rows x 64 reduction entries, 16 B per thread per pass.
    // Two register sets (areg / slab): while stage s is multiplied out of LDS, stage s+1 sits in
    // registers waiting to be dequantized into the other LDS buffer and stage s+2 is in flight.
    const int arow = t >> 3, acol = (t & 7) * 8;
    const int voff_a = (arow * RED + acol) * 2;
    const int astride = APASS * RED * 2;
    uint4_t areg[2][NA];
    auto load_a = [&](uint4_t* dst, int red0) {
#pragma unroll
        for (int i = 0; i < NA; ++i) dst[i] = buf_load128(rs_a, voff_a + i * astride, red0 * 2);
    };
    auto store_a = [&](const uint4_t* src, half_t* dst) {
#pragma unroll
        for (int i = 0; i < NA; ++i)
            *reinterpret_cast<uint4_t*>(dst + (arow + APASS * i) * LDS_STRIDE + acol) = src[i];
    };

    using Slab = typename std::conditional<FWD, FwdSlab<GIDX, NT, BNT>, BwdSlab<GIDX, NT, SZ == 2, BNT>>::type;
    constexpr int NSL = Slab::kSlices;
    Slab slab[2];
    slab[0].init(t, a, c0);
    slab[1].init(t, a, c0);
    typename Slab::Prep prep;

    // bias of this lane's two output columns, requested before everything else: its latency hides under the
    // prologue instead of sitting in the epilogue
    float bias_v[2] = {0.f, 0.f};
    if (FWD && a.bias) {
#pragma unroll
        for (int j = 0; j < 2; ++j) bias_v[j] = (float)a.bias[c0 + wn * 64 + 32 * j + (lane & 31)];
    }

    float16_t acc[TM][2];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int lr = lane & 31, lk = (lane >> 5) * 8;
    const int a_off = (wm * WROWS + lr) * LDS_STRIDE + lk;
    const int b_off = (wn * 64 + lr) * LDS_STRIDE + lk;
    auto read_frags = [&](half8_t* af, half8_t* bf, const half_t* pa, const half_t* pb, int ks) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
            af[i] = *reinterpret_cast<const half8_t*>(pa + a_off + 32 * i * LDS_STRIDE + 16 * ks);
#pragma unroll
        for (int j = 0; j < 2; ++j)
            bf[j] = *reinterpret_cast<const half8_t*>(pb + b_off + 32 * j * LDS_STRIDE + 16 * ks);
    };

    half8_t af[2][TM], bf[2][2];              // operand fragments, double buffered over the sub-steps

    // One pipeline step, branch-free.  CUR = LDS buffer / register set of the stage being multiplied:
    //   registers[CUR]   <- global loads of stage s+2 (clamped to the last stage: a harmless reload)
    //   LDS[CUR^1]       <- dequantized stage s+1 from registers[CUR^1]
    //   acc              += LDS[CUR] (stage s); on entry af[0]/bf[0] already hold sub-step 0
    auto step = [&](int s, auto cur_tag) {
        constexpr int CUR = decltype(cur_tag)::value;
        constexpr int NM = TM * 2 * KS;                        // MFMAs per step
        constexpr int BAR = NM - 3;                   // MFMA index after which the barrier sits (NM-2 .. NM-5 measured: within 3 %)
        // Side work of a step: NL global loads (stage s+2 -> register set CUR) and NC consumer items
        // (stage s+1: register set CUR^1 -> LDS[CUR^1]; NSL dequantization slices with the NA activation
        // stores spread evenly among them).  One load per MFMA slot from slot 0 on (never a burst: eight
        // wavefronts issuing ten loads each at once stall on the address unit), the consumers spread over
        // slots 0..BAR-2 so that the last LDS stores have two MFMAs to drain before the barrier.
        constexpr int NLS = (SZ == 1 && CUR == 1) ? Slab::kLoads - 2 : Slab::kLoads;   // SZ 1: odd steps load no scale / zero
        constexpr int NL = NLS + NA, NC = NSL + NA;
        constexpr int SLOTS = BAR - 1;
        static_assert(SLOTS >= 1, "too few MFMAs per step");
        // fragment set 0 is reloaded right after the barrier: every MFMA of sub-step KS-2 (its last
        // user in this step) must have been issued by then
        static_assert(BAR >= (KS - 1) * TM * 2 - 1, "barrier placed before the last use of fragment set 0");
        const int red_next2 = red_of(s + 2, sr, tm.phase);
        const int red_next1 = red_of(s + 1, sr, tm.phase);
        const half_t* const a_cur = CUR ? sA1 : sA0;
        const half_t* const b_cur = CUR ? sB1 : sB0;
        half_t* const a_nxt = CUR ? sA0 : sA1;
        half_t* const b_nxt = CUR ? sB0 : sB1;
        static_for<0, NM>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            constexpr int ks = i / (TM * 2), r = i % (TM * 2), ti = r / 2, tj = r % 2;
            if constexpr (r == 0 && ks + 1 < KS)
                read_frags(af[(ks + 1) & 1], bf[(ks + 1) & 1], a_cur, b_cur, ks + 1);
            acc[ti][tj] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[ks & 1][ti], bf[ks & 1][tj], acc[ti][tj], 0, 0, 0);
            // (scale, zero) terms of the stage dequantized in this step, in the shadow of the step's first MFMA;
            // SZ 1: the odd stage (CUR == 0) shares the group of the even stage before it
            if constexpr (i == 0 && (SZ != 1 || CUR == 1)) prep = slab[CUR ^ 1].make_prep(c0);
            // load l goes out in slot l*SLOTS/NL (rounded down), consumer q in slot q*SLOTS/NC (rounded up)
            static_for<0, NL>([&](auto lc) {
                constexpr int l = decltype(lc)::value;
                if constexpr (l * SLOTS / NL == i) {
                    if constexpr (l < NLS) slab[CUR].template load_part<l>(a, rs, red_next2);
                    else areg[CUR][l - NLS] = buf_load128(rs_a, voff_a + (l - NLS) * astride, red_next2 * 2);
                }
            });
            constexpr int q_lo = i < SLOTS ? (i * NC + SLOTS - 1) / SLOTS : NC;
            constexpr int q_hi = i < SLOTS ? ((i + 1) * NC + SLOTS - 1) / SLOTS : NC;
            static_for<q_lo, q_hi>([&](auto qc) {
                constexpr int q = decltype(qc)::value;
                constexpr int na_before = q * NA / NC;                       // activation stores among items 0..q-1
                constexpr bool is_a = (q + 1) * NA / NC > na_before;
                if constexpr (is_a)
                    *reinterpret_cast<uint4_t*>(a_nxt + (arow + APASS * na_before) * LDS_STRIDE + acol) = areg[CUR ^ 1][na_before];
                else
                    slab[CUR ^ 1].template store_slice<q - na_before>(a, c0, red_next1, b_nxt, prep);
            });
            if constexpr (i == BAR) {
                // every wavefront has finished reading LDS[CUR] (the last fragments were fetched at
                // sub-step KS-2) and has written its share of LDS[CUR^1]
                __syncthreads();
                read_frags(af[0], bf[0], a_nxt, b_nxt, 0);
                if constexpr (SZ == 2) slab[CUR].fetch_tab(sz_tab, red_next2);   // for the slices of the next step
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    // rank-R adapter step: activations [M, R] (columns beyond R are zero) and the adapter matrix go through the LDS
    // buffers pa / pb like one more reduction step
    auto lora_step = [&](half_t* pa, half_t* pb) {
        __syncthreads();
        const rsrc_t rs_l = make_rsrc(a.la + (size_t)m0 * a.R, (unsigned)rows_valid * (unsigned)a.R * 2u);
#pragma unroll
        for (int i = 0; i < NA; ++i) {
            uint4_t v = {0u, 0u, 0u, 0u};
            if (acol < a.R) v = buf_load128(rs_l, ((arow + APASS * i) * a.R + acol) * 2, 0);
            *reinterpret_cast<uint4_t*>(pa + (arow + APASS * i) * LDS_STRIDE + acol) = v;
        }
        slab[0].store_lora(a, c0, pb, t);
        __syncthreads();
        for (int ks = 0; ks < (a.R + 15) / 16; ++ks) {
            read_frags(af[0], bf[0], pa, pb, ks);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[0][i], bf[0][j], acc[i][j], 0, 0, 0);
        }
    };
    const bool lora_here = a.R > 0 && zsplit == 0;
    const bool lora_masked = lora_here && a.drop.thr15 != 0;              // uniform

    const int red0 = red_of(0, sr, tm.phase), red1 = red_of(1, sr, tm.phase);
    // Same order as inside a step (weights, scale, zero, then the activations): the compiler's wait counts at the
    // head of the main loop are the merge of this path and the loop's own, and with the activations of stage 1
    // requested BEFORE its weights that merge makes every even step wait for ALL loads of the step before it.
    slab[0].load(a, rs, c0, red0);
    load_a(areg[0], red0);
    slab[1].load(a, rs, c0, red1);
    load_a(areg[1], red1);
    if constexpr (SZ == 2) {
        // table of the tile's group: per unit of 8 columns one 16-byte load of scales and one zero word in, four
        // (s_a, s_b, zero_a, zero_b) entries out
        const int g = c0 / a.groupsize;
        for (int u = t; u < (a.N >> 3); u += NT) {
            const uint4_t s8 = buf_load128(rs.s, u * 16, g * a.N * 2);
            const uint32_t z8 = buf_load32(rs.z, u * 4, g * (a.N >> 3) * 4);
            const uint32_t sw[4] = {s8.x, s8.y, s8.z, s8.w};
            uint32_t e[8];
#pragma unroll
            for (int pp = 0; pp < 4; ++pp) {
                e[2 * pp] = sw[pp];
                e[2 * pp + 1] = as_u32(zero_term(as_half2(sw[pp]), (z8 >> (8 * pp)) & 0xFu, (z8 >> (8 * pp + 4)) & 0xFu));
            }
            *reinterpret_cast<uint4_t*>(sz_tab + u * 32) = uint4_t{e[0], e[1], e[2], e[3]};
            *reinterpret_cast<uint4_t*>(sz_tab + u * 32 + 16) = uint4_t{e[4], e[5], e[6], e[7]};
        }
        __syncthreads();
        slab[0].fetch_tab(sz_tab, red0);
        slab[1].fetch_tab(sz_tab, red1);
    }
    if (lora_masked) {
        // Dropout on the adapter input: the adapter's share of out[m, c] exists only where the mask keeps (m, c).
        // So the adapter step runs FIRST, into the zeroed accumulators (through the second pair of LDS buffers,
        // while the loads of the first two stages are in flight), the accumulators are masked, and the main
        // loop adds the unmasked product on top.  The kept values carry 1/(1-p) through lb_scale.
        lora_step(sA1, sB1);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm * WROWS + 32 * i + 8 * (r >> 2) + (lane >> 5) * 4 + (r & 3);
                const uint32_t key = drop_row_key(a.drop, (uint32_t)m);
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int col = c0 + wn * 64 + 32 * j + (lane & 31);
                    const uint32_t w = drop_word(a.drop, key, (uint32_t)col >> 1);
                    if (((w >> (16 * (col & 1))) & 0x7FFFu) < a.drop.thr15) acc[i][j][r] = 0.f;
                }
            }
    }
    store_a(areg[0], sA0);
    prep = slab[0].make_prep(c0);
    static_for<0, NSL>([&](auto jc) { slab[0].template store_slice<decltype(jc)::value>(a, c0, red0, sB0, prep); });
    __syncthreads();
    read_frags(af[0], bf[0], sA0, sB0, 0);
    for (int s = 0; s + 1 < sr.cnt; s += 2) {
        step(s, std::integral_constant<int, 0>{});
        step(s + 1, std::integral_constant<int, 1>{});
    }
    if (sr.cnt & 1) step(sr.cnt - 1, std::integral_constant<int, 0>{});   // an even number of steps precedes it: LDS[0]
    if (lora_here && !lora_masked) lora_step(sA0, sB0);

    // epilogue: acc[i][j][r] is row 8*(r/4) + 4*(lane/32) + r%4, column lane%32 of its 32x32 tile.
    // Each wavefront transposes one 32 x 64 block at a time through its own 4.5 KB of LDS
    // (row stride 72 halves) and writes it as 16-byte pieces: 8 lanes cover one 128-byte row segment.
    const int lc = lane & 31, lrow = (lane >> 5) * 4;
    if (nsplit > 1) {
        // split-K: fp32 partial sums straight from the accumulators (32 lanes cover one 128-byte row segment);
        // the bias rides with split 0, the reduction kernel adds the splits in order and rounds once
        float* const pz = a.part + (size_t)zpart * a.M * a.part_cols - (size_t)a.col_tile0 * BNT;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int col = c0 + wn * 64 + 32 * j + lc;
                const float bv = zsplit == 0 ? bias_v[j] : 0.f;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m = m0 + wm * WROWS + 32 * i + 8 * (r >> 2) + lrow + (r & 3);
                    if (m < a.M) pz[(size_t)m * a.part_cols + col] = acc[i][j][r] + bv;
                }
            }
        return;
    }
    __syncthreads();
    half_t* stage = sA0 + wave * (32 * LDS_STRIDE);
    const int orow = lane >> 3, ocol = (lane & 7) * 8;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const float bv = bias_v[j];
#pragma unroll
            for (int r = 0; r < 16; ++r)
                stage[(8 * (r >> 2) + lrow + (r & 3)) * LDS_STRIDE + 32 * j + lc] = (half_t)(acc[i][j][r] + bv);
        }
        // wavefront-private staging area: a workgroup barrier is not needed, only completion of
        // this wavefront's own LDS writes (the compiler inserts the lgkmcnt wait for the reads)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int rr = orow + 8 * p;
            const int m = m0 + wm * WROWS + 32 * i + rr;
            const uint4_t v = *reinterpret_cast<const uint4_t*>(stage + rr * LDS_STRIDE + ocol);
            if (m < a.M) *reinterpret_cast<uint4_t*>(a.out + (size_t)m * NOUT + c0 + wn * 64 + ocol) = v;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

// FWD: out[M, NOUT=N], reduction length RED=K.   BWD: out[M, NOUT=K], reduction length RED=N.
template <int BM, int WGM, bool FWD, bool GIDX, int SZ = 0, int WGN = 2>
__global__ __launch_bounds__(64 * WGM * WGN) void gemm_kernel(GemmArgs a) {
    const StepRange sr = split_steps((FWD ? a.K : a.N) / BK, blockIdx.z, gridDim.z);
    gemm_body<BM, WGM, FWD, GIDX, SZ, WGN>(a, map_tile(a.phase_step, sr.cnt, a.col_tile0), sr, blockIdx.z, gridDim.z,
                                           blockIdx.z);
}

// Up to kGemmGroup layers that share M, K, the group size and (forward) the activations -- q|k|v, gate|up -- in ONE
// grid, each on its own tensors.
//   forward:    blockIdx.x walks the column tiles of layer 0, then of layer 1, ...; every workgroup computes one tile of
//               one layer's own output, over the whole reduction (no split).
//   grad-input: dx = sum_i dy_i @ W_i^T.  The layers are the "splits" of one launch: blockIdx.z = layer * zs + share,
//               every workgroup leaves an fp32 partial tile (adapter term and dropout mask of ITS layer included) and
//               the ordered reduction adds them all into dx: one launch and one reduction instead of one of each per
//               layer plus the additions of the per-layer results.
constexpr int kGemmGroup = 4;
struct GemmGroupArgs {
    GemmArgs layer[kGemmGroup];
    int tile_end[kGemmGroup];          // forward: running total of column tiles (tile width of the launch)
    int zs;                            // grad-input: reduction shares per layer
};

template <int BM, int WGM, bool FWD, bool GIDX, int SZ = 0, int WGN = 2>
__global__ __launch_bounds__(64 * WGM * WGN) void gemm_group_kernel(GemmGroupArgs g) {
    if constexpr (FWD) {
        const GemmArgs& a0 = g.layer[0];
        const StepRange sr = split_steps(a0.K / BK, 0, 1);
        TileMap tm = map_tile(a0.phase_step, sr.cnt, 0);
        const int li = (tm.tile_c >= g.tile_end[0]) + (tm.tile_c >= g.tile_end[1]) + (tm.tile_c >= g.tile_end[2]);   // uniform
        tm.tile_c -= li == 0 ? 0 : g.tile_end[li - 1];
        const GemmArgs a = g.layer[li];
        gemm_body<BM, WGM, FWD, GIDX, SZ, WGN>(a, tm, sr, 0, 1, 0);
    } else {
        const int li = blockIdx.z / g.zs, zz = blockIdx.z - li * g.zs;
        const GemmArgs a = g.layer[li];
        const StepRange sr = split_steps(a.N / BK, zz, g.zs);
        gemm_body<BM, WGM, FWD, GIDX, SZ, WGN>(a, map_tile(a.phase_step, sr.cnt, 0), sr, zz, gridDim.z, blockIdx.z);
    }
}

// out fp16 [n] = sum over the splits of part[s][n], added in order (bit-reproducible), rounded once.
__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(const float* __restrict__ part, half_t* __restrict__ out,
                                                                 long total, int splits) {
    const long i = ((long)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= total) return;                       // total is a multiple of 4 (NOUT % 128 == 0)
    float4_t v = *reinterpret_cast<const float4_t*>(part + i);
    for (int s = 1; s < splits; ++s) {
        const float4_t u = *reinterpret_cast<const float4_t*>(part + (size_t)s * total + i);
        v[0] += u[0]; v[1] += u[1]; v[2] += u[2]; v[3] += u[3];
    }
    half4_t h = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
    *reinterpret_cast<half4_t*>(out + i) = h;
}

// The same for partial sums that cover only the columns [col0, col0 + part_cols) of the output rows.
__global__ __launch_bounds__(256) void gemm_splitk_reduce_cols_kernel(const float* __restrict__ part, half_t* __restrict__ out,
                                                                      int M, int part_cols, int out_cols, int col0, int splits) {
    const long total = (long)M * part_cols;
    const long i = ((long)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= total) return;                       // part_cols is a multiple of 128
    float4_t v = *reinterpret_cast<const float4_t*>(part + i);
    for (int s = 1; s < splits; ++s) {
        const float4_t u = *reinterpret_cast<const float4_t*>(part + (size_t)s * total + i);
        v[0] += u[0]; v[1] += u[1]; v[2] += u[2]; v[3] += u[3];
    }
    const long m = i / part_cols, c = i - m * part_cols;
    half4_t h = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
    *reinterpret_cast<half4_t*>(out + m * out_cols + col0 + c) = h;
}

// One grid of tiles, with the cheapest way of feeding scale and zero that the problem allows (see gemm_kernel).
constexpr size_t kSzTableMax = 48 * 1024;     // dynamic LDS left beside the 108 KB of tile buffers
template <int BM, int WGM, bool FWD, bool GIDX>
static void launch_tiles(const GemmArgs& a, dim3 grid, hipStream_t stream) {
    const dim3 block(128 * WGM);
    if constexpr (!GIDX) {
        if (a.groupsize % 128 == 0) {
            if constexpr (FWD) {
                const int nsteps = a.K / BK, S = (int)grid.z;
                if (nsteps % (2 * S) == 0 && ((a.phase_step & 0xff) % 2) == 0) {
                    hipLaunchKernelGGL((gemm_kernel<BM, WGM, FWD, GIDX, 1>), grid, block, 0, stream, a);
                    return;
                }
            } else {
                const size_t tab = (size_t)a.N * 4;
                static const bool attr_ok = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_kernel<BM, WGM, FWD, GIDX, 2>),
                                                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)kSzTableMax) == hipSuccess;
                if (attr_ok && tab <= kSzTableMax) {
                    hipLaunchKernelGGL((gemm_kernel<BM, WGM, FWD, GIDX, 2>), grid, block, tab, stream, a);
                    return;
                }
            }
        }
    }
    hipLaunchKernelGGL((gemm_kernel<BM, WGM, FWD, GIDX, 0>), grid, block, 0, stream, a);
}

// 256 x 256 tiles (8 wavefronts of 128 x 64): half the activation traffic and 30 % less LDS traffic per MFMA than the
// 256 x 128 tile; for outputs with enough such tiles to fill the CUs.  No split, no second launch; the tile buffers
// take 144 KB of LDS, so the grad-input kernel keeps its per-step scale / zero loads.
template <bool FWD, bool GIDX>
static hipError_t launch_gemm_wide(GemmArgs a, int nout, hipStream_t stream) {
    const dim3 grid(nout / 256, (a.M + 255) / 256, 1), block(512);
    a.col_tile0 = 0;
    a.part_cols = nout;
    if constexpr (FWD && !GIDX) {
        if (a.groupsize % 128 == 0 && (a.K / BK) % 2 == 0 && ((a.phase_step & 0xff) % 2) == 0) {
            hipLaunchKernelGGL((gemm_kernel<256, 2, FWD, GIDX, 1, 4>), grid, block, 0, stream, a);
            return hipGetLastError();
        }
    }
    hipLaunchKernelGGL((gemm_kernel<256, 2, FWD, GIDX, 0, 4>), grid, block, 0, stream, a);
    return hipGetLastError();
}

// tail_cols > 0: the last tail_cols column tiles run as a second launch with the reduction split tail_splits ways
// (the main launch then covers whole rounds of the CUs, and the remainder does not cost a whole round).
template <int BM, int WGM, bool FWD, bool GIDX>
static hipError_t launch_gemm(GemmArgs a, int nout, int splits, int tail_cols, int tail_splits, hipStream_t stream) {
    const int nc = nout / BN, nr = (a.M + BM - 1) / BM;
    a.col_tile0 = 0;
    a.part_cols = nout;
    launch_tiles<BM, WGM, FWD, GIDX>(a, dim3(nc - tail_cols, nr, splits), stream);
    if (splits > 1) {
        const long total = (long)a.M * nout;
        hipLaunchKernelGGL(gemm_splitk_reduce_kernel, dim3((unsigned)((total / 4 + 255) / 256)), dim3(256), 0, stream,
                           a.part, a.out, total, splits);
    }
    if (tail_cols > 0) {
        a.col_tile0 = nc - tail_cols;
        a.part_cols = tail_cols * BN;
        launch_tiles<BM, WGM, FWD, GIDX>(a, dim3(tail_cols, nr, tail_splits), stream);
        const long total = (long)a.M * a.part_cols;
        hipLaunchKernelGGL(gemm_splitk_reduce_cols_kernel, dim3((unsigned)((total / 4 + 255) / 256)), dim3(256), 0, stream,
                           a.part, a.out, a.M, a.part_cols, nout, a.col_tile0 * BN, tail_splits);
    }
    return hipGetLastError();
}

struct GemmPlan {
    int cfg, splits;
    int tail_cols, tail_splits;      // cfg 2 only: column tiles of the split second launch (0: none)
};

template <bool FWD, bool GIDX>
static hipError_t launch_gemm_cfg(const GemmPlan& p, const GemmArgs& a, int nout, hipStream_t stream) {
    switch (p.cfg) {
        case 0: return launch_gemm<128, 2, FWD, GIDX>(a, nout, p.splits, 0, 1, stream);    // 128 x 128, 4 wavefronts of 64 x 64
        case 1: return launch_gemm<256, 2, FWD, GIDX>(a, nout, p.splits, 0, 1, stream);    // 256 x 128, 4 wavefronts of 128 x 64
        case 3: return launch_gemm_wide<FWD, GIDX>(a, nout, stream);                        // 256 x 256, 8 wavefronts of 128 x 64
        default: return launch_gemm<256, 4, FWD, GIDX>(a, nout, p.splits, p.tail_cols, p.tail_splits, stream);   // 256 x 128, 8 wavefronts of 64 x 64
    }
}

// What TileMap is told: row tile r starts its reduction loop kPhaseStep * r steps later; tiles are ordered in groups
// of kRowTilesPerGroup row tiles (measured optimum over the benchmark shapes).
constexpr int kPhaseStep = 2, kRowTilesPerGroup = 2;

// Launch plan shared by q4_launch_gemm and q4_gemm_plan_workspace.  Few output tiles (small M) leave most CUs
// idle while each tile walks the whole reduction: the reduction is then split over gridDim.z workgroups that
// write fp32 partial tiles, about 1.5 workgroups per CU in total.
static GemmPlan plan_gemm(int M, int red, int nout, size_t workspace_bytes) {
    GemmPlan p;
    p.tail_cols = 0; p.tail_splits = 1;
    const int nsteps = red / BK;
    // Tiles of 256 rows (8 wavefronts, one dequantized slab of W for 256 activation rows) do about twice the work per
    // CU and unit of time that 128-row tiles do, so they are used from 129 rows on: as they are when there are more
    // than 128 of them (even 130 of them on 256 CUs beat 260 tiles of 128 rows), otherwise with the reduction split
    // floor(256 / tiles) ways so that every CU gets one workgroup (never more than 256 workgroups: a second, nearly
    // empty round costs more than the split gains).
    const long t256 = (long)(nout / BN) * ((M + 255) / 256);
    int splits = 1;
    // 256 x 256 tiles from 144 of them on (a workgroup does the work of two 256 x 128 ones in about 1.7 times their
    // time), unless their last round would leave more than a fifth of the CUs' slots empty where the narrower tiles
    // fill theirs better: 3072 x (4096 -> 11008) has 516 wide tiles = 3 rounds for 2.02 rounds of work and stays
    // with the narrow ones (270 against 294 us), 4096 rows have 688 (313 against 356 us).
    const long twide = (nout % 256 == 0) ? (long)(nout / 256) * ((M + 255) / 256) : 0;
    if (twide >= 144 &&
        (twide <= 256 || 5 * twide >= 4 * 256 * ((twide + 255) / 256))) {
        p.cfg = 3; p.splits = 1;
        return p;
    }
    if (t256 > 128 && M > 128) {
        p.cfg = 2;
        // More tiles than CUs and a last round that fills at most half of them: the column tiles of that
        // remainder run as a second launch with the reduction split so that it takes a fraction of a round.
        const int nr = (M + 255) / 256;
        const long rem = t256 % 256;
        if (t256 > 256 && rem > 0) {
            const int tcols = (int)((rem + nr - 1) / nr);
            const long tt = (long)tcols * nr;
            int ts = tt <= 128 ? (int)(256 / tt) : 1;
            if (ts > 8) ts = 8;
            while (ts > 1 && nsteps < 8 * ts) --ts;
            if (ts > 1 && (size_t)ts * (size_t)M * (size_t)tcols * BN * sizeof(float) <= workspace_bytes) {
                p.tail_cols = tcols;
                p.tail_splits = ts;
            }
        }
    } else if (t256 <= 128 && M > 128 && nsteps >= 8 * (int)(256 / t256) &&
               (size_t)(256 / t256 > 8 ? 8 : 256 / t256) * (size_t)M * (size_t)nout * sizeof(float) <= workspace_bytes) {
        p.cfg = 2;                                             // only with room for all its partial tiles
        splits = (int)(256 / t256);
        if (splits > 8) splits = 8;
    } else {
        p.cfg = 0;
        const long tiles = (long)(nout / BN) * ((M + 127) / 128);
        if (tiles < 192) {
            splits = (int)((384 + tiles - 1) / tiles);
            if (splits > 8) splits = 8;                        // measured: more splits only add prologues and partial tiles
            if (splits > nsteps / 4) splits = nsteps / 4;      // at least four steps per workgroup
        }
    }
    while (splits > 1 && (size_t)splits * (size_t)M * (size_t)nout * sizeof(float) > workspace_bytes) --splits;
    p.splits = splits < 1 ? 1 : splits;
    return p;
}

}  // namespace q4

extern "C" int q4_launch_splitk_reduce(const float* part, void* out, long total, int splits, hipStream_t stream) {
    hipLaunchKernelGGL(q4::gemm_splitk_reduce_kernel, dim3((unsigned)((total / 4 + 255) / 256)), dim3(256), 0, stream,
                       part, reinterpret_cast<q4::half_t*>(out), total, splits);
    return hipGetLastError() == hipSuccess ? 0 : -4;
}

extern "C" {
int q4_stream_fwd_applicable(int M, int K, int N, int groupsize, int has_gidx);
int q4_launch_stream_fwd(const void* x, const int32_t* qweight, const int32_t* qzeros, const void* scales, int groupsize,
                         const void* bias, void* y, int M, int K, int N, int G, hipStream_t stream);
int q4_stream_dx_applicable(int M, int K, int N, int groupsize, int has_gidx);
int q4_launch_stream_dx(const void* dy, const int32_t* qweight, const int32_t* qzeros, const void* scales, int groupsize,
                        void* dx, int M, int K, int N, int G, hipStream_t stream);
int q4_skinny_applicable(int M, int K, int N, int groupsize, int has_gidx);
size_t q4_skinny_workspace(int M, int K, int N);
int q4_launch_skinny(const void* x, const int32_t* qweight, const int32_t* qzeros, const void* scales, int groupsize,
                     const void* bias, void* y, int M, int K, int N, int G, void* workspace, hipStream_t stream);
int q4_skinny_dx_applicable(int M, int K, int N, int groupsize, int has_gidx);
size_t q4_skinny_dx_workspace(int M, int K, int N);
int q4_launch_skinny_dx(const void* dy, const int32_t* qweight, const int32_t* qzeros, const void* scales, int groupsize,
                        void* dx, int M, int K, int N, int G, void* workspace, hipStream_t stream);
}

extern "C" int q4_launch_gemm(int fwd, const void* act, const int32_t* qweight, const int32_t* qzeros,
                              const void* scales, const int32_t* g_idx, int groupsize, const void* bias,
                              const void* la, const void* lb, int lb_sr, int lb_sc, int lb_is_f32, float lb_scale, int R,
                              void* out, int M, int K, int N, int G, const q4::DropArgs* drop,
                              void* workspace, size_t workspace_bytes, hipStream_t stream) {
    using namespace q4;
    GemmArgs a;
    a.drop = drop ? *drop : DropArgs{0u, 0u, 0u, 1.0f};
    a.a = reinterpret_cast<const half_t*>(act);
    a.qweight = reinterpret_cast<const uint32_t*>(qweight);
    a.qzeros = reinterpret_cast<const uint32_t*>(qzeros);
    a.scales = reinterpret_cast<const half_t*>(scales);
    a.g_idx = g_idx;
    a.groupsize = groupsize;
    a.gs_inv31 = groupsize >= 64 ? (uint32_t)(((1ull << 31) + (uint64_t)(groupsize / 64) - 1) / (uint64_t)(groupsize / 64)) : 0u;
    a.bias = reinterpret_cast<const half_t*>(bias);
    a.la = reinterpret_cast<const half_t*>(la);
    a.lb = lb;
    a.lb_sr = lb_sr; a.lb_sc = lb_sc; a.lb_is_f32 = lb_is_f32; a.lb_scale = lb_scale * a.drop.scale;
    a.R = (la && lb) ? R : 0;
    a.out = reinterpret_cast<half_t*>(out);
    a.M = M; a.K = K; a.N = N; a.G = G;
    a.phase_step = kPhaseStep | (kRowTilesPerGroup << 8);
    const int nout = fwd ? N : K;
    const bool gidx = g_idx != nullptr;
    // some hundred rows of an output that one round of workgroups covers, no adapter: whole-reduction streaming kernels
    if (fwd && a.R == 0 && q4_stream_fwd_applicable(M, K, N, groupsize, gidx))
        return q4_launch_stream_fwd(act, qweight, qzeros, scales, groupsize, bias, out, M, K, N, G, stream);
    // 17..64 rows, forward, no adapter: the weight-streaming kernel (one pass over the packed weights)
    if (fwd && a.R == 0 && q4_skinny_applicable(M, K, N, groupsize, gidx) && workspace &&
        workspace_bytes >= q4_skinny_workspace(M, K, N))
        return q4_launch_skinny(act, qweight, qzeros, scales, groupsize, bias, out, M, K, N, G, workspace, stream);
    if (!fwd && a.R == 0 && q4_stream_dx_applicable(M, K, N, groupsize, gidx))
        return q4_launch_stream_dx(act, qweight, qzeros, scales, groupsize, out, M, K, N, G, stream);
    // 17..48 rows, grad-input, no adapter: its transposed counterpart
    if (!fwd && a.R == 0 && q4_skinny_dx_applicable(M, K, N, groupsize, gidx) && workspace &&
        workspace_bytes >= q4_skinny_dx_workspace(M, K, N))
        return q4_launch_skinny_dx(act, qweight, qzeros, scales, groupsize, out, M, K, N, G, workspace, stream);
    // tile configuration: 256-row tiles once they still give every CU a workgroup; split-K for few tiles
    const GemmPlan p = plan_gemm(M, fwd ? K : N, nout, workspace ? workspace_bytes : 0);
    a.part = reinterpret_cast<float*>(workspace);
    hipError_t e;
    if (fwd) e = gidx ? launch_gemm_cfg<true, true>(p, a, nout, stream) : launch_gemm_cfg<true, false>(p, a, nout, stream);
    else e = gidx ? launch_gemm_cfg<false, true>(p, a, nout, stream) : launch_gemm_cfg<false, false>(p, a, nout, stream);
    return e == hipSuccess ? 0 : -4;
}

// ---- several layers in one launch (sequential groups only) ---------------------------------------------------------
namespace q4 {
struct GroupPlan { int cfg; int zs; };      // cfg as in launch_gemm_cfg (0: 128 x 128, 2: 256 x 128, 3: 256 x 256); -1: not applicable

// Forward: one tile of one layer per workgroup, no split, so the launch needs enough tiles by itself.
// Grad-input: every layer is a share of the reduction (times zs shares per layer when the tiles are few).
static GroupPlan plan_gemm_group(int fwd, int n, int M, int K, const int* N) {
    GroupPlan p{-1, 1};
    if (n < 2 || n > kGemmGroup || M <= 128) return p;
    const int nr = (M + 255) / 256;
    if (fwd) {
        long tot = 0;
        bool all256 = true;
        for (int i = 0; i < n; ++i) { tot += N[i]; all256 = all256 && N[i] % 256 == 0; }
        const long twide = all256 ? (tot / 256) * nr : 0, t256 = (tot / BN) * nr;
        if (twide >= 144 && (twide <= 256 || 5 * twide >= 4 * 256 * ((twide + 255) / 256))) p.cfg = 3;
        else if (t256 >= 192) p.cfg = 2;
        return p;
    }
    const long twide = K % 256 == 0 ? (long)(K / 256) * nr * n : 0, t256 = (long)(K / BN) * nr * n;
    if (twide >= 144 && twide <= 256) { p.cfg = 3; return p; }
    p.cfg = 2;
    if (t256 < 192) {
        int mn = N[0];
        for (int i = 1; i < n; ++i) mn = N[i] < mn ? N[i] : mn;
        if (mn / BK >= 16) p.zs = 2;                     // at least eight steps per workgroup
    }
    return p;
}

template <int BM, int WGM, bool FWD, int WGN>
static void launch_group_tiles(const GemmGroupArgs& g, int n, dim3 grid, hipStream_t stream) {
    const GemmArgs& a = g.layer[0];
    const dim3 block(64 * WGM * WGN);
    if (a.groupsize % 128 == 0) {
        if constexpr (FWD) {
            if ((a.K / BK) % 2 == 0 && ((a.phase_step & 0xff) % 2) == 0) {
                hipLaunchKernelGGL((gemm_group_kernel<BM, WGM, FWD, false, 1, WGN>), grid, block, 0, stream, g);
                return;
            }
        } else if constexpr (WGN == 2) {
            int mx = 0;
            for (int i = 0; i < n; ++i) mx = g.layer[i].N > mx ? g.layer[i].N : mx;
            const size_t tab = (size_t)mx * 4;
            static const bool attr_ok = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_group_kernel<BM, WGM, FWD, false, 2, WGN>),
                                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)kSzTableMax) == hipSuccess;
            if (attr_ok && tab <= kSzTableMax) {
                hipLaunchKernelGGL((gemm_group_kernel<BM, WGM, FWD, false, 2, WGN>), grid, block, tab, stream, g);
                return;
            }
        }
    }
    hipLaunchKernelGGL((gemm_group_kernel<BM, WGM, FWD, false, 0, WGN>), grid, block, 0, stream, g);
}
}  // namespace q4

extern "C" int q4_gemm_group_applicable(int fwd, int n, int M, int K, const int* N) {
    return q4::plan_gemm_group(fwd, n, M, K, N).cfg >= 0;
}

extern "C" size_t q4_gemm_group_plan_workspace(int fwd, int n, int M, int K, const int* N) {
    const q4::GroupPlan p = q4::plan_gemm_group(fwd, n, M, K, N);
    if (fwd || p.cfg < 0) return 0;
    return (size_t)n * p.zs * (size_t)M * (size_t)K * sizeof(float);
}

// act: forward the shared x (act[i] may all be the same pointer), grad-input dy_i.  out: forward y_i, grad-input out[0] = dx.
extern "C" int q4_launch_gemm_group(int fwd, int n, const void* const* act, const int32_t* const* qweight,
                                    const int32_t* const* qzeros, const void* const* scales, int groupsize,
                                    const void* const* bias, const void* const* la, const void* const* lb, const int* lb_sr,
                                    const int* lb_sc, const int* lb_is_f32, const float* lb_scale, const int* R,
                                    void* const* out, int M, int K, const int* N, const q4::DropArgs* const* drop,
                                    void* workspace, size_t workspace_bytes, hipStream_t stream) {
    using namespace q4;
    const GroupPlan p = plan_gemm_group(fwd, n, M, K, N);
    if (p.cfg < 0) return -2;
    const size_t need = fwd ? 0 : (size_t)n * p.zs * (size_t)M * (size_t)K * sizeof(float);
    if (need > 0 && (!workspace || workspace_bytes < need)) return -3;
    GemmGroupArgs g;
    const int tile_w = p.cfg == 3 ? 256 : BN;
    int tiles = 0;
    for (int i = 0; i < kGemmGroup; ++i) {
        const int j = i < n ? i : n - 1;                // unused slots repeat the last layer (never selected)
        GemmArgs& a = g.layer[i];
        a.drop = (drop && drop[j]) ? *drop[j] : DropArgs{0u, 0u, 0u, 1.0f};
        a.a = reinterpret_cast<const half_t*>(act[j]);
        a.qweight = reinterpret_cast<const uint32_t*>(qweight[j]);
        a.qzeros = reinterpret_cast<const uint32_t*>(qzeros[j]);
        a.scales = reinterpret_cast<const half_t*>(scales[j]);
        a.g_idx = nullptr;
        a.groupsize = groupsize;
        a.gs_inv31 = (uint32_t)(((1ull << 31) + (uint64_t)(groupsize / 64) - 1) / (uint64_t)(groupsize / 64));
        a.bias = fwd && bias ? reinterpret_cast<const half_t*>(bias[j]) : nullptr;
        a.la = la ? reinterpret_cast<const half_t*>(la[j]) : nullptr;
        a.lb = lb ? lb[j] : nullptr;
        a.R = (a.la && a.lb) ? R[j] : 0;
        a.lb_sr = a.R ? lb_sr[j] : 0; a.lb_sc = a.R ? lb_sc[j] : 0; a.lb_is_f32 = a.R ? lb_is_f32[j] : 0;
        a.lb_scale = (a.R ? lb_scale[j] : 0.f) * a.drop.scale;
        a.out = reinterpret_cast<half_t*>(fwd ? out[j] : out[0]);
        a.M = M; a.K = K; a.N = N[j]; a.G = (K + groupsize - 1) / groupsize;
        a.phase_step = kPhaseStep | (kRowTilesPerGroup << 8);
        a.part = reinterpret_cast<float*>(workspace);
        a.col_tile0 = 0;
        a.part_cols = fwd ? N[j] : K;
        if (i < n) tiles += N[i] / tile_w;
        g.tile_end[i] = i < n ? tiles : 0x7fffffff;
    }
    g.zs = p.zs;
    const int bm = p.cfg == 0 ? 128 : 256;
    const int nr = (M + bm - 1) / bm;
    const dim3 grid(fwd ? tiles : K / tile_w, nr, fwd ? 1 : n * p.zs);
    if (fwd) {
        if (p.cfg == 3) launch_group_tiles<256, 2, true, 4>(g, n, grid, stream);
        else launch_group_tiles<256, 4, true, 2>(g, n, grid, stream);
    } else {
        if (p.cfg == 3) launch_group_tiles<256, 2, false, 4>(g, n, grid, stream);
        else launch_group_tiles<256, 4, false, 2>(g, n, grid, stream);
        const long total = (long)M * K;
        hipLaunchKernelGGL(gemm_splitk_reduce_kernel, dim3((unsigned)((total / 4 + 255) / 256)), dim3(256), 0, stream,
                           g.layer[0].part, g.layer[0].out, total, n * p.zs);
    }
    return hipGetLastError() == hipSuccess ? 0 : -4;
}

// Workspace that lets q4_launch_gemm use its preferred split for this shape (0: no split wanted).
extern "C" size_t q4_gemm_plan_workspace(int fwd, int M, int K, int N) {
    using namespace q4;
    const int nout = fwd ? N : K;
    const GemmPlan p = plan_gemm(M, fwd ? K : N, nout, ~(size_t)0);
    size_t need = p.splits > 1 ? (size_t)p.splits * (size_t)M * (size_t)nout * sizeof(float) : 0;
    if (p.tail_cols > 0) need = (size_t)p.tail_splits * (size_t)M * (size_t)p.tail_cols * BN * sizeof(float);
    if (fwd && M > 16 && M <= 64) {               // the skinny kernel's partial rows (it may or may not apply)
        const size_t sk = q4_skinny_workspace(M, K, N);
        if (sk > need) need = sk;
    }
    if (!fwd && M > 16 && M <= 48) {
        const size_t sk = q4_skinny_dx_workspace(M, K, N);
        if (sk > need) need = sk;
    }
    return need;
}
