"""Generates tests/golden/q4_golden.npz: small packed GPTQ layers with the dense fp16 weight
and matmul results the reference arithmetic must give.

The reference's own tests hold no vector for this path (they need a downloaded 7B checkpoint),
and the reference cannot be imported or built here (no nvcc, no peft/colorama).  The expected
values are therefore produced by an implementation that shares NOTHING with oracle/:
pure-Python loops that follow the reference kernel's thread-index arithmetic
(quant_cuda_kernel.cu:1127-1153: h, b, w, n_rows, z_rows, z_cols, z_shift, i, shift) with exact
rational arithmetic (fractions.Fraction) and a hand-written round-to-nearest-even to binary16.
Matmul expectations are exact rational sums of the dequantized values, stored as float64.

tests/golden/q4_golden_f32.npz holds the same for the kernel's float instantiation (fp32 scales, fp32 result), from
exact rational arithmetic and a round-to-nearest-even to binary32 written for it.

Run:  python tests/golden/make_fixtures.py     (about a minute; --f32-only writes the float file alone)
"""
import os
import struct
from fractions import Fraction

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
BLOCKWIDTH, BLOCKHEIGHT4 = 128, 16        # quant_cuda_kernel.cu:179-183


def half_bits_to_fraction(h: int) -> Fraction:
    sign = -1 if (h >> 15) & 1 else 1
    exp = (h >> 10) & 0x1F
    man = h & 0x3FF
    assert exp != 31, "fixtures use finite values only"
    if exp == 0:
        return sign * Fraction(man, 1 << 24)
    return sign * Fraction((1 << 10) + man, 1 << 10) * (Fraction(2) ** (exp - 15))


def rn16(v: Fraction) -> int:
    """Exact rational -> nearest binary16 bit pattern, ties to even, overflow to inf."""
    if v == 0:
        return 0
    sign = 0x8000 if v < 0 else 0
    a = -v if v < 0 else v
    # find e with 2^e <= a < 2^(e+1)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    if Fraction(2) ** (e + 1) <= a:
        e += 1
    e = max(e, -14)                                  # subnormals share the exponent of 2^-14
    q = a / (Fraction(2) ** (e - 10))                # in units of the last place
    n = q.numerator // q.denominator
    rem = q - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (n & 1)):
        n += 1
    if n >= (1 << 11):                               # carried into the next binade
        n >>= 1
        e += 1
    if e > 15:
        return sign | 0x7C00
    if n < (1 << 10):                                # subnormal (only possible with e == -14)
        return sign | n
    return sign | ((e + 15) << 10) | (n - (1 << 10))


def as_unsigned(i: int) -> int:
    return i & 0xFFFFFFFF


def recons_v2_reference_loops(qweight, qzeros, scales_bits, g_idx):
    """One Python iteration per CUDA thread of VecQuant4ReconsV2Kernel<Half>."""
    height, width = qweight.shape                    # :1160-1161
    zero_width = qzeros.shape[1]
    out = np.zeros((height * 8, width), dtype=np.uint16)
    for bx in range((height + BLOCKHEIGHT4 - 1) // BLOCKHEIGHT4):
        for by in range((width + BLOCKWIDTH - 1) // BLOCKWIDTH):
            for b in range(BLOCKWIDTH):
                for tx in range(BLOCKWIDTH):
                    h = BLOCKHEIGHT4 * bx
                    w = BLOCKWIDTH * by + tx
                    n_rows = h * 8 + b
                    n_cols = w
                    if n_rows >= height * 8 or n_cols >= width:
                        continue                     # the reference has no such guard; shapes here are multiples of 128
                    z_rows = int(g_idx[n_rows])
                    z_cols = n_cols // 8
                    z_shift = (n_cols % 8) * 4
                    scale = half_bits_to_fraction(int(scales_bits[z_rows, n_cols]))
                    z = (as_unsigned(int(qzeros[z_rows, z_cols])) >> z_shift) & 0xF
                    zero = half_bits_to_fraction(rn16(scale * (z + 1)))
                    i_row = h + b // 8
                    shift = b % 8 * 4
                    tmp = as_unsigned(int(qweight[i_row, w]))
                    q = (tmp >> shift) & 0xF
                    prod = half_bits_to_fraction(rn16(scale * q))
                    out[n_rows, n_cols] = rn16(prod - zero)
    return out


def make_case(seed, K, N, groupsize, act_order, M):
    rng = np.random.default_rng(seed)
    G = K // groupsize
    codes = rng.integers(0, 16, size=(K, N))
    zc = rng.integers(0, 16, size=(G, N))
    qweight = np.zeros((K // 8, N), dtype=np.int64)
    for k in range(K):
        qweight[k // 8] |= codes[k] << (4 * (k % 8))
    qzeros = np.zeros((G, N // 8), dtype=np.int64)
    for n in range(N):
        qzeros[:, n // 8] |= zc[:, n] << (4 * (n % 8))
    to_i32 = lambda a: np.array([struct.unpack("<i", struct.pack("<I", int(v)))[0] for v in a.ravel()],
                                dtype=np.int32).reshape(a.shape)
    qweight, qzeros = to_i32(qweight), to_i32(qzeros)
    scales = rng.uniform(0.005, 0.02, size=(G, N)).astype(np.float16)
    if act_order:
        perm = rng.permutation(K)
        g_idx = np.empty(K, dtype=np.int32)
        g_idx[perm] = (np.arange(K) // groupsize).astype(np.int32)
    else:
        g_idx = (np.arange(K) // groupsize).astype(np.int32)
    W_bits = recons_v2_reference_loops(qweight, qzeros, scales.view(np.uint16), g_idx)
    x = rng.standard_normal((M, K)).astype(np.float16)
    dy = rng.standard_normal((M, N)).astype(np.float16)
    Wf = [[half_bits_to_fraction(int(b)) for b in row] for row in W_bits]
    xf = [[half_bits_to_fraction(int(b)) for b in row] for row in x.view(np.uint16)]
    dyf = [[half_bits_to_fraction(int(b)) for b in row] for row in dy.view(np.uint16)]
    y = np.array([[float(sum(xf[m][k] * Wf[k][n] for k in range(K))) for n in range(N)] for m in range(M)])
    dx = np.array([[float(sum(dyf[m][n] * Wf[k][n] for n in range(N))) for k in range(K)] for m in range(M)])
    return dict(qweight=qweight, qzeros=qzeros, scales=scales, g_idx=g_idx, W_bits=W_bits, x=x, dy=dy, y=y, dx=dx,
                codes=codes.astype(np.uint8), zcodes=zc.astype(np.uint8))


# ------------------------------------------------------------------------------------------------ float flavour
def float_bits_to_fraction(u: int) -> Fraction:
    sign = -1 if (u >> 31) & 1 else 1
    exp = (u >> 23) & 0xFF
    man = u & 0x7FFFFF
    assert exp != 255, "fixtures use finite values only"
    if exp == 0:
        return sign * Fraction(man, 1 << 149)
    return sign * Fraction((1 << 23) + man, 1 << 23) * (Fraction(2) ** (exp - 127))


def rn32(v: Fraction) -> int:
    """Exact rational -> nearest binary32 bit pattern, ties to even (written on its own, not derived from rn16:
    it scales to an integer significand first and rounds the integer)."""
    if v == 0:
        return 0
    sign = 0x80000000 if v < 0 else 0
    a = abs(v)
    e = max(a.numerator.bit_length() - a.denominator.bit_length() - 2, -126)      # a lower bound of floor(log2 a)
    while Fraction(2) ** (e + 1) <= a:
        e += 1                                        # subnormals keep the exponent -126
    ulp = Fraction(2) ** (e - 23)
    n, twice_rem = divmod(2 * (a / ulp), 2)
    n = int(n)
    if twice_rem > 1 or (twice_rem == 1 and n % 2 == 1):
        n += 1
    if n == (1 << 24):
        n, e = 1 << 23, e + 1
    assert e <= 127, "fixtures stay finite"
    if n < (1 << 23):
        return sign | n
    return sign | ((e + 127) << 23) | (n - (1 << 23))


def recons_v2_float(s: Fraction, q: int, z: int):
    """(fused, separate) bit patterns of VecQuant4ReconsV2Kernel<float> for one element
    (quant_cuda_kernel.cu:1146-1151): zero = rn32(s * (z + 1)); result = s * q - zero, which nvcc's default
    contraction evaluates as one fma (one rounding); the separately rounded form is kept beside it."""
    zero = float_bits_to_fraction(rn32(s * (z + 1)))
    fused = rn32(s * q - zero)
    separate = rn32(float_bits_to_fraction(rn32(s * q)) - zero)
    return fused, separate


def main_f32():
    out = {}
    rng = np.random.default_rng(11)
    # scale bit patterns: typical GPTQ magnitudes with all 23 fraction bits in play, plus edge patterns
    typical = rng.uniform(0.003, 0.03, size=160).astype(np.float32).view(np.uint32)
    wide = (rng.integers(100, 140, size=60).astype(np.uint32) << 23) | rng.integers(0, 1 << 23, size=60).astype(np.uint32)
    edge = np.array([0x00000001, 0x007FFFFF, 0x00800000, 0x3F800000, 0x3FFFFFFF, 0x80000001, 0xBF800000, 0x7B7FFFFF],
                    dtype=np.uint32)
    sb = np.concatenate([typical, wide, edge]).astype(np.uint32)
    fused = np.zeros((sb.size, 16, 16), dtype=np.uint32)
    separate = np.zeros_like(fused)
    for i, u in enumerate(sb):
        S = float_bits_to_fraction(int(u))
        for q in range(16):
            for z in range(16):
                fused[i, q, z], separate[i, q, z] = recons_v2_float(S, q, z)
    out["scalar_scale_bits"] = sb
    out["scalar_fused"] = fused
    out["scalar_separate"] = separate
    # one small act-order layer, thread-index arithmetic as in recons_v2_reference_loops
    K, N, groupsize = 128, 64, 32
    G = K // groupsize
    codes = rng.integers(0, 16, size=(K, N))
    zc = rng.integers(0, 16, size=(G, N))
    qweight = np.zeros((K // 8, N), dtype=np.int64)
    for k in range(K):
        qweight[k // 8] |= codes[k] << (4 * (k % 8))
    qzeros = np.zeros((G, N // 8), dtype=np.int64)
    for n in range(N):
        qzeros[:, n // 8] |= zc[:, n] << (4 * (n % 8))
    qweight = qweight.astype(np.uint32).view(np.int32)
    qzeros = qzeros.astype(np.uint32).view(np.int32)
    scales = rng.uniform(0.003, 0.03, size=(G, N)).astype(np.float32)
    perm = rng.permutation(K)
    g_idx = np.empty(K, dtype=np.int32)
    g_idx[perm] = (np.arange(K) // groupsize).astype(np.int32)
    W = np.zeros((K, N), dtype=np.uint32)
    sbits = scales.view(np.uint32)
    for n_rows in range(K):
        for n_cols in range(N):
            z_rows = int(g_idx[n_rows])
            z = (as_unsigned(int(qzeros[z_rows, n_cols // 8])) >> ((n_cols % 8) * 4)) & 0xF
            q = (as_unsigned(int(qweight[n_rows // 8, n_cols])) >> (n_rows % 8 * 4)) & 0xF
            W[n_rows, n_cols] = recons_v2_float(float_bits_to_fraction(int(sbits[z_rows, n_cols])), q, z)[0]
    out.update(layer_qweight=qweight, layer_qzeros=qzeros, layer_scales=scales, layer_g_idx=g_idx, layer_W_bits=W)
    np.savez_compressed(os.path.join(HERE, "q4_golden_f32.npz"), **out)
    print("wrote", os.path.join(HERE, "q4_golden_f32.npz"))


def main():
    out = {}
    for name, kw in (("seq", dict(seed=101, K=256, N=128, groupsize=128, act_order=False, M=2)),
                     ("actorder", dict(seed=202, K=256, N=128, groupsize=128, act_order=True, M=2))):
        case = make_case(**kw)
        for k, v in case.items():
            out[f"{name}_{k}"] = v
    # scalar known answers: (scale bits, q, z) -> W bits, incl. cases where rounding order matters
    rng = np.random.default_rng(7)
    sb = np.concatenate([rng.integers(0x1C00, 0x2800, size=200), [0x0001, 0x03FF, 0x0400, 0x3C00, 0x6BFF, 0x8001, 0xBC00]])
    tab = np.zeros((sb.size, 16, 16), dtype=np.uint16)
    for i, s in enumerate(sb):
        S = half_bits_to_fraction(int(s))
        for q in range(16):
            for z in range(16):
                zero = half_bits_to_fraction(rn16(S * (z + 1)))
                prod = half_bits_to_fraction(rn16(S * q))
                tab[i, q, z] = rn16(prod - zero)
    out["scalar_scale_bits"] = sb.astype(np.uint16)
    out["scalar_table"] = tab
    np.savez_compressed(os.path.join(HERE, "q4_golden.npz"), **out)
    print("wrote", os.path.join(HERE, "q4_golden.npz"))


if __name__ == "__main__":
    import sys
    if "--f32-only" not in sys.argv:
        main()
    main_f32()
