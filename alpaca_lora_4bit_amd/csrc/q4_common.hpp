// Shared device helpers for the gfx950 4-bit GPTQ kernels.
//
// Layout being decoded (reference: src/alpaca_lora_4bit/quant_cuda/quant_cuda_kernel.cu:1138-1152):
//   qweight[k/8, n] holds the code of row k in bits 4*(k%8)..4*(k%8)+3,
//   qzeros[g, n/8] holds the zero code of column n in bits 4*(n%8)..,
//   W[k,n] = rn16( rn16(s*q) - rn16(s*(z+1)) ) with s = scales[g,n].
// All fp16 arithmetic that must reproduce those three roundings is written on _Float16
// vectors and this code is compiled with -ffp-contract=off, so a multiply is never fused
// with the subtraction that follows it.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace q4 {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));

constexpr uint32_t kMagic = 0x64006400u;  // two fp16 1024.0: (0x6400 | q) == 1024 + q exactly

__device__ __forceinline__ half2_t as_half2(uint32_t u) {
    return __builtin_bit_cast(half2_t, u);
}
__device__ __forceinline__ uint32_t as_u32(half2_t h) {
    return __builtin_bit_cast(uint32_t, h);
}

// (lo | hi << 16) of two 4-bit codes -> two fp16 values equal to the codes (exact).
__device__ __forceinline__ half2_t codes_to_half2(uint32_t packed_codes) {
    const half2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f};
    return as_half2(packed_codes | kMagic) - k1024;
}

// Three-rounding dequant of a pair: rn16(rn16(s*q) - zero), zero = rn16(s*(z+1)) precomputed.
__device__ __forceinline__ half2_t dequant_pair(half2_t q, half2_t s, half2_t zero) {
    half2_t p = s * q;
    return p - zero;
}

// zero term rn16(s * half(z+1)) for two columns.
__device__ __forceinline__ half2_t zero_term(half2_t s, uint32_t z_lo, uint32_t z_hi) {
    half2_t zp1 = {(half_t)(float)(z_lo + 1u), (half_t)(float)(z_hi + 1u)};
    return s * zp1;
}

// Natural-order unpack of one packed word (eight codes e0..e7 of one column) into four
// half2 registers (e0,e1) (e2,e3) (e4,e5) (e6,e7), each value exactly the code.
__device__ __forceinline__ void unpack8_natural(uint32_t w, half2_t out[4]) {
    const uint32_t lo = w & 0x0F0F0F0Fu;          // bytes e0 e2 e4 e6
    const uint32_t hi = (w >> 4) & 0x0F0F0F0Fu;   // bytes e1 e3 e5 e7
    // v_perm_b32 byte selectors: 0-3 pick from the 2nd operand, 4-7 from the 1st, 0x0c = 0x00.
    out[0] = codes_to_half2(__builtin_amdgcn_perm(hi, lo, 0x0c040c00u));
    out[1] = codes_to_half2(__builtin_amdgcn_perm(hi, lo, 0x0c050c01u));
    out[2] = codes_to_half2(__builtin_amdgcn_perm(hi, lo, 0x0c060c02u));
    out[3] = codes_to_half2(__builtin_amdgcn_perm(hi, lo, 0x0c070c03u));
}

// Buffer-resource loads: a 32-bit byte offset per lane plus a uniform byte offset; an access
// past `bytes` returns zero instead of faulting, so tiles need no per-lane bounds branches.
constexpr int kRsrcFlags = 0x00020000;
typedef __amdgpu_buffer_rsrc_t rsrc_t;

__device__ __forceinline__ rsrc_t make_rsrc(const void* p, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, kRsrcFlags);
}
__device__ __forceinline__ uint4_t buf_load128(rsrc_t r, int voff, int soff) {
    return __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0));
}
// Same with the non-temporal cache policy, for data that is read once (packed weights in the streaming kernels).
constexpr int kAuxNonTemporal = 2;
__device__ __forceinline__ uint4_t buf_load128_stream(rsrc_t r, int voff, int soff) {
    return __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, kAuxNonTemporal));
}
__device__ __forceinline__ uint2_t buf_load64(rsrc_t r, int voff, int soff) {
    return __builtin_bit_cast(uint2_t, __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, 0));
}
__device__ __forceinline__ uint32_t buf_load32(rsrc_t r, int voff, int soff) {
    return __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0);
}
__device__ __forceinline__ uint32_t buf_load16(rsrc_t r, int voff, int soff) {
    return (uint32_t)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(r, voff, soff, 0);
}

// ---- counter-based dropout mask ----------------------------------------------------------------------------
// The adapter input of Linear4bitLt is dropout(x) (src/alpaca_lora_4bit/models.py:66).  Nothing is stored for it:
// element (row, col) of x is dropped iff a 15-bit draw that is a pure function of (seed, row, col) is below
// thr15 = round(p * 32768), so forward (xa = dropout(x) @ A^T) and backward (dA = dyb^T @ dropout(x), and the
// adapter's share of dx masked the same way) regenerate the same mask.  One 32-bit word serves the column pair
// (2*pair, 2*pair + 1): bits 0..14 and 16..30.  The mixer is the "lowbias32" finalizer.
struct DropArgs {
    uint32_t seed_lo, seed_hi;
    uint32_t thr15;           // 0: dropout off
    float scale;              // 1 / (1 - thr15 / 32768): applied by the kernels to what survives
};
__device__ __forceinline__ uint32_t drop_row_key(const DropArgs& d, uint32_t row) { return row * 0x9E3779B1u + d.seed_lo; }
__device__ __forceinline__ uint32_t drop_word(const DropArgs& d, uint32_t row_key, uint32_t pair) {
    uint32_t h = row_key ^ (pair * 0x85EBCA6Bu + d.seed_hi);
    h ^= h >> 16; h *= 0x7FEB352Du;
    h ^= h >> 15; h *= 0x846CA68Bu;
    h ^= h >> 16;
    return h;
}
// 0xFFFF in the 16-bit half of a kept element, 0x0000 in that of a dropped one.  thr_pair = thr15 | thr15 << 16;
// draws and threshold are 15-bit, so the signed 16-bit differences cannot overflow.
typedef short short2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t drop_keep_mask(uint32_t word, uint32_t thr_pair) {
    const short2_t v = __builtin_bit_cast(short2_t, word & 0x7FFF7FFFu);
    const short2_t dropped = (v - __builtin_bit_cast(short2_t, thr_pair)) >> 15;    // all ones where draw < thr
    return ~__builtin_bit_cast(uint32_t, dropped);
}
__device__ __forceinline__ bool drop_keeps(const DropArgs& d, uint32_t row, uint32_t col) {
    const uint32_t w = drop_word(d, drop_row_key(d, row), col >> 1);
    return ((w >> (16 * (col & 1))) & 0x7FFFu) >= d.thr15;
}

}  // namespace q4
