"""CPU oracle for the 4-bit GPTQ dequant-matmul path (numpy).

TEST INFRASTRUCTURE ONLY.  Nothing in the product package imports this file; it is
the checker used by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg
of bench.py.  It restates, in plain numpy, the arithmetic of the reference
(johnsmith0031/alpaca_lora_4bit); every function cites the reference lines it
follows.  Paths are relative to the reference checkout.

Parity status of each function (what pins it is in tests/test_oracle_*.py):

  unpack_qweight / unpack_qzeros / pack_*   pinned  (hand-written nibble vectors, sign-bit
                                                     nibble, round trip, pure-Python index loop)
  rn16 arithmetic of dequant_v2             pinned  (exact Fraction arithmetic + an independent
                                                     Fraction-based round-to-nearest-even,
                                                     closed forms s=1,z=0 and q=z+1, a case where
                                                     the three-rounding and one-rounding forms differ)
  dequant_v2 act-order                      pinned  (row-permutation invariant, brute-force loop)
  matmul_recons / matmul_recons_t           pinned  (integer-exact brute force, linearity,
                                                     transpose identity)
  gemv_v2_fp32                              pinned  (same brute force; fp32 form)
  lora_forward / lora_backward              pinned  (finite differences in float64, and torch
                                                     autograd through dense nn.Linear in tests)
  dequant_v1 / dequant2_v2                  pinned  (exact Fraction arithmetic with the independent
                                                     round-to-nearest-even of tests/golden/make_fixtures.py,
                                                     pure-Python index loops for the 2-bit packing)
  dequant_v2_f32                            pinned  (exact Fraction arithmetic with a round-to-binary32 of its own,
                                                     tests/golden/q4_golden_f32.npz: scalar table over all (q, z),
                                                     an act-order layer, and cases where fused != separate)
  peft 0.6 LoraLayer internals              parity unpinned (peft is not importable here; only the
                                                     arithmetic in models.py:58-66 is restated)
"""
from __future__ import annotations

import numpy as np

MAXQ = 15
PACK = 8  # 4-bit codes per int32 word


# --------------------------------------------------------------------------- layout
def pack_qweight(codes: np.ndarray) -> np.ndarray:
    """codes uint8 [K, N] (0..15) -> qweight int32 [K/8, N].

    Row k lives in word k // 8 at bit offset 4 * (k % 8): the inverse of the unpack at
    src/alpaca_lora_4bit/quant_cuda/quant_cuda_kernel.cu:1148-1151
    (i = width*h + width*(b/8) + w; shift = b % 8 * 4).
    """
    codes = np.asarray(codes)
    K, N = codes.shape
    assert K % PACK == 0
    c = codes.astype(np.uint32).reshape(K // PACK, PACK, N)
    word = np.zeros((K // PACK, N), dtype=np.uint32)
    for j in range(PACK):
        word |= (c[:, j, :] & 0xF) << np.uint32(4 * j)
    return word.view(np.int32)


def pack_qzeros(zcodes: np.ndarray) -> np.ndarray:
    """zcodes uint8 [G, N] (0..15) -> qzeros int32 [G, N/8].

    Column n lives in word n // 8 at bit offset 4 * (n % 8): inverse of
    quant_cuda_kernel.cu:1144-1147 (z_cols = n_cols / 8; z_shift = (n_cols % 8) * 4).
    """
    zcodes = np.asarray(zcodes)
    G, N = zcodes.shape
    assert N % PACK == 0
    c = zcodes.astype(np.uint32).reshape(G, N // PACK, PACK)
    word = np.zeros((G, N // PACK), dtype=np.uint32)
    for j in range(PACK):
        word |= (c[:, :, j] & 0xF) << np.uint32(4 * j)
    return word.view(np.int32)


def unpack_qweight(qweight: np.ndarray) -> np.ndarray:
    """qweight int32 [K/8, N] -> codes uint8 [K, N]; quant_cuda_kernel.cu:1148-1151.

    The word is reinterpreted as unsigned before shifting (as_unsigned, :185-187), so a
    code >= 8 in the top nibble (sign bit set) must still come out as 8..15.
    """
    w = np.ascontiguousarray(qweight).view(np.uint32)
    KW, N = w.shape
    out = np.empty((KW, PACK, N), dtype=np.uint8)
    for j in range(PACK):
        out[:, j, :] = (w >> np.uint32(4 * j)) & 0xF
    return out.reshape(KW * PACK, N)


def unpack_qzeros(qzeros: np.ndarray) -> np.ndarray:
    """qzeros int32 [G, N/8] -> zero codes uint8 [G, N]; quant_cuda_kernel.cu:1144-1147."""
    w = np.ascontiguousarray(qzeros).view(np.uint32)
    G, NW = w.shape
    out = np.empty((G, NW, PACK), dtype=np.uint8)
    for j in range(PACK):
        out[:, :, j] = (w >> np.uint32(4 * j)) & 0xF
    return out.reshape(G, NW * PACK)


# --------------------------------------------------------------------------- dequant
def dequant_v2(qweight, qzeros, scales, g_idx) -> np.ndarray:
    """Dense fp16 W [K, N] exactly as VecQuant4ReconsV2Kernel<Half> produces it.

    quant_cuda_kernel.cu:1127-1153:  g = g_idx[k]; scale = scales[g, n];
    zero = scale * Half(z + 1); result = scale * Half(q) - zero, each operator rounding
    to fp16, i.e.  W = rn16( rn16(s*q) - rn16(s*(z+1)) ).
    numpy float16 operators compute in float32 and round once per operator, which is the
    same thing (an 11x11-bit product is exact in float32; float32 -> float16 double rounding
    of a sum of two halves is innocuous because 24 >= 2*11 + 2).
    """
    scales = np.asarray(scales)
    assert scales.dtype == np.float16
    q = unpack_qweight(qweight)                       # [K, N]
    z = unpack_qzeros(qzeros)                         # [G, N]
    g = np.asarray(g_idx).astype(np.int64)            # [K]
    K, N = q.shape
    assert g.shape == (K,) and z.shape[1] == N and scales.shape == z.shape
    s_rows = scales[g]                                # [K, N] fp16
    zp1 = (z.astype(np.int32) + 1).astype(np.float16)[g]
    zero = s_rows * zp1                               # rn16(s*(z+1))
    prod = s_rows * q.astype(np.float16)              # rn16(s*q)
    return prod - zero                                # rn16(prod - zero)


def dequant_v1(qweight, scales, zeros) -> np.ndarray:
    """Dense fp16 W of a v1 layer as VecQuant4ReconsV1Kernel<Half> produces it
    (quant_cuda_kernel.cu:1076-1097): scale, zero per column; result = scale * Half(q) - zero,
    i.e. W = rn16( rn16(s*q) - zero ).  Parity pinned by exact-rational arithmetic in tests/test_oracle.py."""
    s = np.asarray(scales).reshape(-1)
    z = np.asarray(zeros).reshape(-1)
    assert s.dtype == np.float16 and z.dtype == np.float16
    q = unpack_qweight(qweight).astype(np.float16)
    return (s[None, :] * q) - z[None, :]


def pack_qweight2(codes: np.ndarray) -> np.ndarray:
    """codes uint8 [K, N] in 0..3 -> int32 [K/16, N]: row k in bits 2*(k%16).. of word [k/16, n]
    (index arithmetic of quant_cuda_kernel.cu:1206-1208)."""
    K, N = codes.shape
    c = codes.astype(np.uint32).reshape(K // 16, 16, N)
    w = np.zeros((K // 16, N), dtype=np.uint32)
    for e in range(16):
        w |= c[:, e, :] << np.uint32(2 * e)
    return w.view(np.int32)


def pack_qzeros2(zcodes: np.ndarray) -> np.ndarray:
    """zero codes uint8 [G, N] in 0..3 -> int32 [G, N/16]: column n in bits 2*(n%16).. of word [g, n/16]
    (quant_cuda_kernel.cu:1201-1203)."""
    G, N = zcodes.shape
    c = zcodes.astype(np.uint32).reshape(G, N // 16, 16)
    w = np.zeros((G, N // 16), dtype=np.uint32)
    for e in range(16):
        w |= c[:, :, e] << np.uint32(2 * e)
    return w.view(np.int32)


def dequant2_v2(qweight, qzeros, scales, g_idx) -> np.ndarray:
    """Dense fp16 W of a 2-bit v2 layer as VecQuant2ReconsV2Kernel<Half> produces it
    (quant_cuda_kernel.cu:1185-1211): the 4-bit formula with 2-bit fields,
    W = rn16( rn16(s*q) - rn16(s*(z+1)) )."""
    scales = np.asarray(scales)
    assert scales.dtype == np.float16
    wq = np.asarray(qweight).view(np.uint32)
    zq = np.asarray(qzeros).view(np.uint32)
    K, N = wq.shape[0] * 16, wq.shape[1]
    k = np.arange(K)
    q = ((wq[k // 16, :] >> ((k % 16) * 2).astype(np.uint32)[:, None]) & 3).astype(np.float16)      # [K, N]
    n = np.arange(N)
    z = ((zq[:, n // 16] >> ((n % 16) * 2).astype(np.uint32)[None, :]) & 3).astype(np.int32)         # [G, N]
    g = np.asarray(g_idx).astype(np.int64)
    s_rows = scales[g]
    zero = s_rows * (z + 1).astype(np.float16)[g]
    return s_rows * q - zero


def dequant_v2_f32(qweight, qzeros, scales, g_idx, fused=True) -> np.ndarray:
    """Dense fp32 W [K, N] as VecQuant4ReconsV2Kernel<float> produces it (fp32 scales; the dispatch on
    scales.type() at quant_cuda_kernel.cu:1173-1181 instantiates the template of :1126-1152 for float).

    zero = rn32(s * (z + 1)); result = s * q - zero.  nvcc contracts a * b - c into one fma by default and the
    reference's setup.py passes no flag, so the built kernel rounds once: rn32(s*q - zero) (fused=True).  float64
    holds s*q (24 + 4 bits) and its difference with a float32 of nearby exponent exactly, so one cast to float32
    is that single rounding.  fused=False rounds the product first (what the source says without contraction).
    """
    scales = np.asarray(scales)
    assert scales.dtype == np.float32
    q = unpack_qweight(qweight)
    z = unpack_qzeros(qzeros)
    g = np.asarray(g_idx).astype(np.int64)
    s_rows = scales[g]
    zero = s_rows * (z.astype(np.int32) + 1).astype(np.float32)[g]            # rn32(s*(z+1))
    if fused:
        return (s_rows.astype(np.float64) * q.astype(np.float64) - zero.astype(np.float64)).astype(np.float32)
    return s_rows * q.astype(np.float32) - zero


def dequant_v2_single_rounding(qweight, qzeros, scales, g_idx) -> np.ndarray:
    """The OTHER order, (q - (z+1)) * s with one rounding (triton_utils.py:85-95).

    Not the parity target; kept so tests can show that the two orders are distinguishable
    and that the HIP kernels implement the three-rounding one.
    """
    q = unpack_qweight(qweight).astype(np.float32)
    z = unpack_qzeros(qzeros).astype(np.float32)
    g = np.asarray(g_idx).astype(np.int64)
    s = np.asarray(scales).astype(np.float32)
    return ((q - (z[g] + 1.0)) * s[g]).astype(np.float16)


# --------------------------------------------------------------------------- matmul
def matmul_recons(x, qweight, qzeros, scales, g_idx) -> np.ndarray:
    """y = x @ W with fp32 accumulation, W = dequant_v2(...).

    matmul_utils_4bit.py:114-124 (_matmul4bit_v2_recons, transpose=False): recons into a
    dense fp16 buffer, then torch.matmul(x, buffer).  Returned in float32 (the
    fp32-accumulated result the tolerance is defined against); callers round to fp16.
    """
    W = dequant_v2(qweight, qzeros, scales, g_idx).astype(np.float32)
    x = np.asarray(x)
    assert x.shape[-1] == W.shape[0]                  # matmul_utils_4bit.py:118
    return x.astype(np.float32) @ W


def matmul_recons_t(dy, qweight, qzeros, scales, g_idx) -> np.ndarray:
    """dx = dy @ W.T (matmul_utils_4bit.py:125-126, transpose=True; autograd_4bit.py:53)."""
    W = dequant_v2(qweight, qzeros, scales, g_idx).astype(np.float32)
    dy = np.asarray(dy)
    assert dy.shape[-1] == W.shape[1]                 # matmul_utils_4bit.py:120
    return dy.astype(np.float32) @ W.T


def gemv_v2_fp32(x, qweight, qzeros, scales, g_idx) -> np.ndarray:
    """VecQuant4MatMulKernel<float> numerics (quant_cuda_kernel.cu:475-536): everything in
    fp32, per-row g_idx, w = s*q - s*(z+1) with fp32 roundings, y = sum_k w*x.
    Summation order in the reference is non-deterministic (atomicAdd, :535); float64
    accumulation here gives the value the tolerance is measured from.
    """
    q = unpack_qweight(qweight).astype(np.float32)
    z = unpack_qzeros(qzeros).astype(np.float32)
    g = np.asarray(g_idx).astype(np.int64)
    s = np.asarray(scales).astype(np.float32)[g]
    w = (s * q - s * (z[g] + np.float32(1.0))).astype(np.float32)
    return (np.asarray(x).astype(np.float64) @ w.astype(np.float64)).astype(np.float32)


# --------------------------------------------------------------------------- LoRA
def lora_forward(x, W, A, B, scaling, bias=None, keep=None, drop_scale=1.0) -> np.ndarray:
    """Linear4bitLt.forward (models.py:51-69) for one active adapter:
    result = x @ W (+ bias, autograd_4bit.py:206-207) + lora_B(lora_A(dropout(x))) * scaling,
    with lora_A.weight = A [r, K], lora_B.weight = B [N, r].  float64 throughout.
    `keep` [M, K] (0/1) and `drop_scale` = 1/(1-p) describe the dropout of models.py:63-66 as torch's nn.Dropout
    applies it in training mode: dropout(x) = x * keep * drop_scale; keep=None is dropout off / eval mode.
    """
    x = np.asarray(x, dtype=np.float64)
    y = x @ np.asarray(W, dtype=np.float64)
    if bias is not None:
        y = y + np.asarray(bias, dtype=np.float64)
    xd = x if keep is None else x * np.asarray(keep, dtype=np.float64) * float(drop_scale)
    xa = xd @ np.asarray(A, dtype=np.float64).T
    return y + (xa @ np.asarray(B, dtype=np.float64).T) * float(scaling)


def lora_backward(x, dy, W, A, B, scaling, keep=None, drop_scale=1.0):
    """Gradients of lora_forward w.r.t. x, A, B (closed form of what torch autograd
    computes over autograd_4bit.py:45-54 plus models.py:66).  float64.  With xd = x * keep * drop_scale
    (dropout in front of lora_A; keep=None: xd = x, mask = 1):
      dx = dy @ W.T + keep * drop_scale * (scaling * (dy @ B) @ A)
      dA = scaling * (dy @ B).T @ xd         [r, K]
      dB = scaling * dy.T @ (xd @ A.T)       [N, r]
    """
    x = np.asarray(x, dtype=np.float64)
    dy = np.asarray(dy, dtype=np.float64)
    W = np.asarray(W, dtype=np.float64)
    A = np.asarray(A, dtype=np.float64)
    B = np.asarray(B, dtype=np.float64)
    s = float(scaling)
    m = 1.0 if keep is None else np.asarray(keep, dtype=np.float64) * float(drop_scale)
    xd = x * m
    dyB = dy @ B
    dx = dy @ W.T + m * (s * (dyB @ A))
    dA = s * (dyB.T @ xd)
    dB = s * (dy.T @ (xd @ A.T))
    return dx, dA, dB


def dropout_keep_counter(M, C, seed, p):
    """(keep uint8 [M, C], scale): the counter-based dropout mask the library documents in include/q4_gptq.h
    (no reference counterpart: the reference's mask comes from torch's generator, models.py:63 -- any mask with
    the right statistics is a valid nn.Dropout).  Restated here from the header's formula with numpy uint32
    arithmetic: element (m, c) is kept iff its 15-bit draw >= round(p * 32768)."""
    thr = min(int(np.float32(p) * np.float32(32768.0) + np.float32(0.5)), 32767)
    seed_lo, seed_hi = np.uint32(seed & 0xFFFFFFFF), np.uint32((seed >> 32) & 0xFFFFFFFF)
    with np.errstate(over="ignore"):
        rows = np.arange(M, dtype=np.uint32)[:, None]
        pairs = np.arange(C // 2, dtype=np.uint32)[None, :]
        w = (rows * np.uint32(0x9E3779B1) + seed_lo) ^ (pairs * np.uint32(0x85EBCA6B) + seed_hi)
        w ^= w >> np.uint32(16)
        w = w * np.uint32(0x7FEB352D)
        w ^= w >> np.uint32(15)
        w = w * np.uint32(0x846CA68B)
        w ^= w >> np.uint32(16)
    keep = np.empty((M, C), dtype=np.uint8)
    keep[:, 0::2] = (w & np.uint32(0x7FFF)) >= thr
    keep[:, 1::2] = ((w >> np.uint32(16)) & np.uint32(0x7FFF)) >= thr
    return keep, 32768.0 / (32768 - thr)


# --------------------------------------------------------------------------- synthetic data
def make_layer(K, N, groupsize=128, act_order=False, seed=0):
    """Seeded synthetic GPTQ layer: codes and zero codes ~ U{0..15}, scales ~ U[0.005, 0.02]
    fp16, g_idx[k] = k // groupsize, or (act_order) a random permutation mapped to groups so
    that each group owns exactly `groupsize` scattered rows.
    Buffer shapes/dtypes as registered at autograd_4bit.py:181-189.
    """
    rng = np.random.default_rng(seed)
    G = (K + groupsize - 1) // groupsize
    codes = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    zcodes = rng.integers(0, 16, size=(G, N), dtype=np.uint8)
    scales = rng.uniform(0.005, 0.02, size=(G, N)).astype(np.float16)
    if act_order:
        perm = rng.permutation(K)
        g_idx = np.empty(K, dtype=np.int32)
        g_idx[perm] = (np.arange(K) // groupsize).astype(np.int32)
    else:
        g_idx = (np.arange(K) // groupsize).astype(np.int32)
    return dict(qweight=pack_qweight(codes), qzeros=pack_qzeros(zcodes), scales=scales,
                g_idx=g_idx, codes=codes, zcodes=zcodes, K=K, N=N, G=G, groupsize=groupsize)


def make_activations(M, K, seed=0):
    rng = np.random.default_rng(seed + 1000003)
    return rng.standard_normal((M, K)).astype(np.float16)


def make_lora(K, N, r=8, seed=0):
    """A [r, K] Kaiming-uniform(a=sqrt(5)) -> U(-1/sqrt(K), 1/sqrt(K)); B [N, r] ~ N(0, 0.02)."""
    rng = np.random.default_rng(seed + 2000003)
    bound = 1.0 / np.sqrt(K)
    A = rng.uniform(-bound, bound, size=(r, K)).astype(np.float32)
    B = (rng.standard_normal((N, r)) * 0.02).astype(np.float32)
    return A, B
