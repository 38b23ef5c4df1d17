"""Pins the CPU oracle (oracle/q4_oracle.py, q4_oracle.c, q4_torch.py) WITHOUT the GPU.

What fixes the oracle, since the reference holds no runnable vector for this path:
  * tests/golden/q4_golden.npz, produced by exact-rational pure-Python loops that follow the
    reference kernel's index arithmetic (tests/golden/make_fixtures.py) and share no code with oracle/;
  * closed forms (s=1,z=0 -> q-1; q=z+1 -> 0), a hand-computed three-rounding case, the sign-bit nibble;
  * invariants (pack/unpack round trip, act-order == row permutation, linearity, transpose identity);
  * agreement of three independent implementations (numpy, C with its own fp16 rounding, torch).
"""
import os

import numpy as np
import pytest

from oracle import c_oracle, q4_oracle as o

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "q4_golden.npz"))


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint16)


# ------------------------------------------------------------------ golden fixtures
@pytest.mark.parametrize("case", ["seq", "actorder"])
def test_dequant_matches_golden(case):
    args = [GOLD[f"{case}_{k}"] for k in ("qweight", "qzeros", "scales", "g_idx")]
    want = GOLD[f"{case}_W_bits"]
    assert np.array_equal(_bits(o.dequant_v2(*args)), want)
    assert np.array_equal(_bits(c_oracle.dequant_v2(*args)), want)
    import torch
    from oracle import q4_torch
    got = q4_torch.dequant_v2(*[torch.from_numpy(a) for a in args]).numpy()
    assert np.array_equal(_bits(got), want)


@pytest.mark.parametrize("case", ["seq", "actorder"])
def test_matmul_matches_golden(case):
    args = [GOLD[f"{case}_{k}"] for k in ("qweight", "qzeros", "scales", "g_idx")]
    x, dy, y, dx = (GOLD[f"{case}_{k}"] for k in ("x", "dy", "y", "dx"))
    assert np.allclose(o.matmul_recons(x, *args), y, rtol=0, atol=2e-5 * np.abs(y).max())
    assert np.allclose(o.matmul_recons_t(dy, *args), dx, rtol=0, atol=2e-5 * np.abs(dx).max())
    W = o.dequant_v2(*args)
    assert np.allclose(c_oracle.matmul(x, W), y, rtol=0, atol=2e-5 * np.abs(y).max())
    assert np.allclose(c_oracle.matmul_t(dy, W), dx, rtol=0, atol=2e-5 * np.abs(dx).max())
    # the fp32 GEMV form differs from the fp16-dequant form only by the dequant roundings
    assert np.abs(o.gemv_v2_fp32(x, *args) - y).max() <= 2e-3 * np.abs(y).max()


def test_scalar_table_matches_golden():
    sb, tab = GOLD["scalar_scale_bits"], GOLD["scalar_table"]
    assert np.array_equal(c_oracle.dequant_table(sb), tab)
    s = sb.view(np.float16)[:, None, None]
    q = np.arange(16, dtype=np.float16)[None, :, None]
    zp1 = (np.arange(16) + 1).astype(np.float16)[None, None, :]
    with np.errstate(all="ignore"):
        got = s * q - s * zp1                      # numpy half ops: one rounding per operator
    assert np.array_equal(_bits(got), tab)


def test_pack_layout_matches_golden_codes():
    for case in ("seq", "actorder"):
        assert np.array_equal(o.unpack_qweight(GOLD[f"{case}_qweight"]), GOLD[f"{case}_codes"])
        assert np.array_equal(o.unpack_qzeros(GOLD[f"{case}_qzeros"]), GOLD[f"{case}_zcodes"])
        assert np.array_equal(o.pack_qweight(GOLD[f"{case}_codes"]), GOLD[f"{case}_qweight"])
        assert np.array_equal(o.pack_qzeros(GOLD[f"{case}_zcodes"]), GOLD[f"{case}_qzeros"])


# ------------------------------------------------------------------ closed forms
def _one_group_layer(codes, zcodes, scale):
    K, N = codes.shape
    return (o.pack_qweight(codes), o.pack_qzeros(zcodes), np.full((1, N), scale, dtype=np.float16),
            np.zeros(K, dtype=np.int32))


def test_unit_scale_zero_code_gives_q_minus_one():
    rng = np.random.default_rng(0)
    codes = rng.integers(0, 16, size=(64, 64), dtype=np.uint8)
    W = o.dequant_v2(*_one_group_layer(codes, np.zeros((1, 64), dtype=np.uint8), 1.0))
    assert np.array_equal(W.astype(np.int32), codes.astype(np.int32) - 1)


def test_code_equal_zero_point_gives_exact_zero():
    rng = np.random.default_rng(1)
    z = rng.integers(0, 15, size=(1, 64), dtype=np.uint8)
    codes = np.repeat(z + 1, 64, axis=0).astype(np.uint8)
    W = o.dequant_v2(o.pack_qweight(codes), o.pack_qzeros(z),
                     rng.uniform(0.005, 0.02, size=(1, 64)).astype(np.float16), np.zeros(64, dtype=np.int32))
    assert not W.any()


def test_golden_table_pins_the_three_rounding_order():
    """The exact-rational golden table is NOT reproduced by the single-rounding form
    (q - (z+1)) * s: a dropped or merged rounding in the oracle would fail the golden tests."""
    sb, tab = GOLD["scalar_scale_bits"], GOLD["scalar_table"]
    s = sb.view(np.float16).astype(np.float32)[:, None, None]
    q = np.arange(16, dtype=np.float32)[None, :, None]
    zp1 = (np.arange(16, dtype=np.float32) + 1)[None, None, :]
    one = ((q - zp1) * s).astype(np.float16)
    frac = (_bits(one) != tab).mean()
    assert frac > 0.1
    # same on a full layer, and the two orders never differ by more than one ulp at |W| < 0.5
    lay = o.make_layer(256, 128, 128, seed=3)
    three = o.dequant_v2(lay["qweight"], lay["qzeros"], lay["scales"], lay["g_idx"])
    one = o.dequant_v2_single_rounding(lay["qweight"], lay["qzeros"], lay["scales"], lay["g_idx"])
    frac = (_bits(three) != _bits(one)).mean()
    assert 0.2 < frac < 0.7
    assert np.abs(three.astype(np.float32) - one.astype(np.float32)).max() <= 2.5e-4


def test_sign_bit_nibble_is_unsigned():
    """Code >= 8 in the top nibble sets the int32 sign bit; an arithmetic shift would smear it."""
    codes = np.zeros((8, 8), dtype=np.uint8)
    codes[7, :] = 15
    qw = o.pack_qweight(codes)
    assert (qw < 0).all()
    assert np.array_equal(o.unpack_qweight(qw), codes)
    z = np.full((1, 8), 9, dtype=np.uint8)
    qz = o.pack_qzeros(z)
    assert (qz < 0).all() and np.array_equal(o.unpack_qzeros(qz), z)


# ------------------------------------------------------------------ invariants
def test_pack_unpack_round_trip_random():
    rng = np.random.default_rng(5)
    codes = rng.integers(0, 16, size=(128, 96), dtype=np.uint8)
    assert np.array_equal(o.unpack_qweight(o.pack_qweight(codes)), codes)
    z = rng.integers(0, 16, size=(4, 96), dtype=np.uint8)
    assert np.array_equal(o.unpack_qzeros(o.pack_qzeros(z)), z)


def test_act_order_equals_row_permutation():
    """Dequant with a permuted g_idx == dequant of the group-sorted layer with rows put back."""
    lay = o.make_layer(512, 64, 128, act_order=True, seed=9)
    W = o.dequant_v2(lay["qweight"], lay["qzeros"], lay["scales"], lay["g_idx"])
    order = np.argsort(lay["g_idx"], kind="stable")
    sorted_codes = lay["codes"][order]
    Ws = o.dequant_v2(o.pack_qweight(sorted_codes), lay["qzeros"], lay["scales"],
                      (np.arange(512) // 128).astype(np.int32))
    assert np.array_equal(_bits(W[order]), _bits(Ws))
    # brute force over every element
    for k in range(0, 512, 37):
        for n in range(0, 64, 5):
            g = lay["g_idx"][k]
            want = c_oracle.lib().q4o_dequant_scalar(int(lay["scales"].view(np.uint16)[g, n]), int(lay["codes"][k, n]),
                                                     int(lay["zcodes"][g, n]))
            assert int(_bits(W)[k, n]) == want


def test_matmul_integer_exact_and_linear():
    """With s = 1 and integer activations every product is an integer: fp32 sums are exact."""
    rng = np.random.default_rng(11)
    codes = rng.integers(0, 16, size=(64, 64), dtype=np.uint8)
    layer = _one_group_layer(codes, np.full((1, 64), 3, dtype=np.uint8), 1.0)
    x = rng.integers(-4, 5, size=(3, 64)).astype(np.float16)
    want = x.astype(np.int64) @ (codes.astype(np.int64) - 4)
    assert np.array_equal(o.matmul_recons(x, *layer).astype(np.int64), want)
    dy = rng.integers(-4, 5, size=(3, 64)).astype(np.float16)
    want_t = dy.astype(np.int64) @ (codes.astype(np.int64) - 4).T
    assert np.array_equal(o.matmul_recons_t(dy, *layer).astype(np.int64), want_t)
    # transpose identity  <dy, x@W> == <dy@W^T, x>
    lay = o.make_layer(256, 128, 128, seed=2)
    args = (lay["qweight"], lay["qzeros"], lay["scales"], lay["g_idx"])
    xx, dd = o.make_activations(4, 256, 1), o.make_activations(4, 128, 2)
    lhs = (dd.astype(np.float64) * o.matmul_recons(xx, *args)).sum()
    rhs = (o.matmul_recons_t(dd, *args) * xx.astype(np.float64)).sum()
    assert abs(lhs - rhs) <= 1e-4 * abs(lhs)


def test_lora_backward_by_finite_differences():
    rng = np.random.default_rng(13)
    K, N, r, M = 12, 10, 3, 5
    W = rng.standard_normal((K, N))
    A, B = rng.standard_normal((r, K)), rng.standard_normal((N, r))
    x, dy = rng.standard_normal((M, K)), rng.standard_normal((M, N))
    dx, dA, dB = o.lora_backward(x, dy, W, A, B, 2.0)
    loss = lambda x_, A_, B_: (o.lora_forward(x_, W, A_, B_, 2.0) * dy).sum()
    eps = 1e-6
    for arr, grad, which in ((x, dx, 0), (A, dA, 1), (B, dB, 2)):
        for idx in [(0, 0), (1, 2), (arr.shape[0] - 1, arr.shape[1] - 1)]:
            p = arr.copy(); p[idx] += eps
            m = arr.copy(); m[idx] -= eps
            args_p = [x, A, B]; args_p[which] = p
            args_m = [x, A, B]; args_m[which] = m
            fd = (loss(*args_p) - loss(*args_m)) / (2 * eps)
            assert abs(fd - grad[idx]) <= 1e-5 * max(1.0, abs(fd))


def test_lora_backward_with_a_dropout_mask_by_finite_differences_and_autograd():
    """The `keep` branch (dropout in front of lora_A, models.py:63-66): the closed-form gradients against central
    differences of lora_forward with the same mask, and against torch autograd through nn.Linear layers fed
    x * keep * scale; a dropped element gets no adapter gradient."""
    import torch
    rng = np.random.default_rng(23)
    K, N, r, M = 12, 10, 4, 6
    W = rng.standard_normal((K, N))
    A, B = rng.standard_normal((r, K)), rng.standard_normal((N, r))
    x, dy = rng.standard_normal((M, K)), rng.standard_normal((M, N))
    keep, scale = o.dropout_keep_counter(M, K, seed=1234567, p=0.4)
    assert keep.shape == (M, K) and 0 < keep.sum() < keep.size and abs(scale - 32768.0 / (32768 - 13107)) < 1e-12
    dx, dA, dB = o.lora_backward(x, dy, W, A, B, 2.0, keep=keep, drop_scale=scale)
    loss = lambda x_, A_, B_: (o.lora_forward(x_, W, A_, B_, 2.0, keep=keep, drop_scale=scale) * dy).sum()
    eps = 1e-6
    for arr, grad, which in ((x, dx, 0), (A, dA, 1), (B, dB, 2)):
        for idx in [(0, 0), (1, 2), (2, 3), (arr.shape[0] - 1, arr.shape[1] - 1)]:
            p = arr.copy(); p[idx] += eps
            m = arr.copy(); m[idx] -= eps
            args_p = [x, A, B]; args_p[which] = p
            args_m = [x, A, B]; args_m[which] = m
            fd = (loss(*args_p) - loss(*args_m)) / (2 * eps)
            assert abs(fd - grad[idx]) <= 1e-5 * max(1.0, abs(fd))
    base_only = dy @ W.T
    dropped = keep == 0
    assert np.allclose(dx[dropped], base_only[dropped])             # no adapter share where x was dropped
    assert not np.allclose(dx[~dropped], base_only[~dropped])
    xt = torch.from_numpy(x.copy()).requires_grad_(True)
    At, Bt = torch.from_numpy(A.copy()).requires_grad_(True), torch.from_numpy(B.copy()).requires_grad_(True)
    xd = xt * torch.from_numpy(keep.astype(np.float64)) * scale
    y = xt @ torch.from_numpy(W) + (xd @ At.t()) @ Bt.t() * 2.0
    y.backward(torch.from_numpy(dy))
    assert np.allclose(y.detach().numpy(), o.lora_forward(x, W, A, B, 2.0, keep=keep, drop_scale=scale))
    assert np.allclose(xt.grad.numpy(), dx) and np.allclose(At.grad.numpy(), dA) and np.allclose(Bt.grad.numpy(), dB)


def test_dropout_keep_counter_statistics_and_determinism():
    """The mask is a pure function of (seed, row, column): repeatable, different for another seed, keeps about 1 - p."""
    k1, s1 = o.dropout_keep_counter(256, 512, seed=42, p=0.05)
    k2, _ = o.dropout_keep_counter(256, 512, seed=42, p=0.05)
    k3, _ = o.dropout_keep_counter(256, 512, seed=43, p=0.05)
    assert np.array_equal(k1, k2) and not np.array_equal(k1, k3)
    assert abs(k1.mean() - 0.95) < 0.005 and abs(s1 - 32768.0 / (32768 - 1638)) < 1e-12
    k0, s0 = o.dropout_keep_counter(8, 16, seed=1, p=0.0)
    assert k0.all() and s0 == 1.0
    assert np.array_equal(o.dropout_keep_counter(300, 512, seed=42, p=0.05)[0][:256], k1)     # rows do not depend on M


def test_lora_forward_matches_torch_autograd():
    """Closed-form gradients == torch autograd through dense nn.Linear layers (models.py:58-66)."""
    import torch
    rng = np.random.default_rng(17)
    K, N, r, M = 16, 24, 8, 6
    W = rng.standard_normal((K, N))
    A, B = rng.standard_normal((r, K)), rng.standard_normal((N, r))
    x, dy = rng.standard_normal((M, K)), rng.standard_normal((M, N))
    base = torch.nn.Linear(K, N, bias=False, dtype=torch.float64)
    la = torch.nn.Linear(K, r, bias=False, dtype=torch.float64)
    lb = torch.nn.Linear(r, N, bias=False, dtype=torch.float64)
    base.weight.data, la.weight.data, lb.weight.data = (torch.from_numpy(W.T.copy()), torch.from_numpy(A.copy()),
                                                        torch.from_numpy(B.copy()))
    xt = torch.from_numpy(x.copy()).requires_grad_(True)
    y = base(xt) + lb(la(xt)) * 2.0
    y.backward(torch.from_numpy(dy))
    dx, dA, dB = o.lora_backward(x, dy, W, A, B, 2.0)
    assert np.allclose(y.detach().numpy(), o.lora_forward(x, W, A, B, 2.0))
    assert np.allclose(xt.grad.numpy(), dx) and np.allclose(la.weight.grad.numpy(), dA)
    assert np.allclose(lb.weight.grad.numpy(), dB)


# ------------------------------------------------------------------ implementations agree
def test_numpy_c_and_torch_agree_on_random_layers():
    import torch
    from oracle import q4_torch
    for seed, act in ((1, False), (2, True)):
        lay = o.make_layer(512, 192, 64, act_order=act, seed=seed)
        args = (lay["qweight"], lay["qzeros"], lay["scales"], lay["g_idx"])
        a = o.dequant_v2(*args)
        assert np.array_equal(_bits(a), _bits(c_oracle.dequant_v2(*args)))
        t = q4_torch.dequant_v2(*[torch.from_numpy(v) for v in args]).numpy()
        assert np.array_equal(_bits(a), _bits(t))


def test_c_oracle_exhaustive_scalar_table_equals_numpy():
    """All 63 488 finite fp16 scales x 16 x 16: the C oracle's own fp16 rounding == numpy's."""
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    fin = bits[np.isfinite(bits.view(np.float16))]
    T = c_oracle.dequant_table(fin)
    s = fin.view(np.float16)[:, None, None]
    q = np.arange(16, dtype=np.float16)[None, :, None]
    zp1 = (np.arange(16) + 1).astype(np.float16)[None, None, :]
    with np.errstate(all="ignore"):
        Tn = s * q - s * zp1
    same = (_bits(Tn) == T) | (np.isnan(Tn) & np.isnan(T.view(np.float16)))
    assert same.all()


def test_synthetic_generators_follow_the_config_distributions():
    lay = o.make_layer(1024, 256, 128, act_order=True, seed=3)
    assert lay["qweight"].shape == (128, 256) and lay["qzeros"].shape == (8, 32) and lay["scales"].shape == (8, 256)
    assert lay["scales"].dtype == np.float16 and 0.005 <= lay["scales"].min() and lay["scales"].max() <= 0.02
    counts = np.bincount(lay["g_idx"], minlength=8)
    assert (counts == 128).all() and not np.array_equal(lay["g_idx"], np.arange(1024) // 128)
    A, B = o.make_lora(4096, 4096, 8, seed=1)
    assert A.shape == (8, 4096) and B.shape == (4096, 8) and np.abs(A).max() <= 1 / 64 and 0.015 < B.std() < 0.025


# --------------------------------------------------------------------------- older layouts (v1, 2-bit)
def _load_generator():
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(os.path.dirname(__file__), "golden", "make_fixtures.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_dequant_v1_against_exact_rational_arithmetic(oracle):
    """W = rn16(rn16(s*q) - zero) per element (quant_cuda_kernel.cu:1094), checked with Fractions and the
    generator's own round-to-nearest-even."""
    gen = _load_generator()
    rng = np.random.default_rng(5)
    K, N = 16, 64
    codes = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    scales = rng.uniform(0.004, 0.03, size=N).astype(np.float16)
    zeros = (scales.astype(np.float32) * rng.integers(1, 17, size=N)).astype(np.float16)
    W = oracle.dequant_v1(oracle.pack_qweight(codes), scales, zeros)
    sb, zb, wb = scales.view(np.uint16), zeros.view(np.uint16), W.view(np.uint16)
    for k in range(K):
        for n in range(N):
            s = gen.half_bits_to_fraction(int(sb[n]))
            prod = gen.half_bits_to_fraction(gen.rn16(s * int(codes[k, n])))
            expect = gen.rn16(prod - gen.half_bits_to_fraction(int(zb[n])))
            assert int(wb[k, n]) == expect or (expect & 0x7FFF) == 0 and (int(wb[k, n]) & 0x7FFF) == 0


def test_dequant2_against_loops_and_exact_arithmetic(oracle):
    """2-bit packing by pure-Python index arithmetic of the kernel (quant_cuda_kernel.cu:1196-1210) and the
    three-rounding value by Fractions."""
    gen = _load_generator()
    rng = np.random.default_rng(6)
    K, N, gs = 64, 64, 32
    G = K // gs
    codes = rng.integers(0, 4, size=(K, N), dtype=np.uint8)
    zc = rng.integers(0, 4, size=(G, N), dtype=np.uint8)
    scales = rng.uniform(0.01, 0.2, size=(G, N)).astype(np.float16)
    g_idx = rng.permutation(K).astype(np.int32) % G                     # scattered groups
    qw, qz = oracle.pack_qweight2(codes), oracle.pack_qzeros2(zc)
    assert qw.shape == (K // 16, N) and qz.shape == (G, N // 16)
    W = oracle.dequant2_v2(qw, qz, scales, g_idx)
    sb, wb = scales.view(np.uint16), W.view(np.uint16)
    for k in range(0, K, 3):
        for n in range(0, N, 5):
            word = gen.as_unsigned(int(qw[k // 16, n]))
            q = (word >> (k % 16 * 2)) & 0x3
            assert q == codes[k, n]
            g = int(g_idx[k])
            z = ((gen.as_unsigned(int(qz[g, n // 16])) >> ((n % 16) * 2)) & 0x3) + 1
            assert z == zc[g, n] + 1
            s = gen.half_bits_to_fraction(int(sb[g, n]))
            zero = gen.half_bits_to_fraction(gen.rn16(s * z))
            prod = gen.half_bits_to_fraction(gen.rn16(s * q))
            expect = gen.rn16(prod - zero)
            assert int(wb[k, n]) == expect or (expect & 0x7FFF) == 0 and (int(wb[k, n]) & 0x7FFF) == 0


# --------------------------------------------------------------------------- float flavour of the dense dequant
GOLD32 = np.load(os.path.join(os.path.dirname(__file__), "golden", "q4_golden_f32.npz"))


def _scalar_layer_f32():
    """A layer holding every (scale, q, z) of the golden table: column n = scale index, row k has q = k % 16,
    groups of 32 rows (the smallest the library takes), one group per zero code."""
    sb = GOLD32["scalar_scale_bits"]
    n_pad = (sb.size + 63) // 64 * 64
    s = np.zeros(n_pad, dtype=np.uint32)
    s[:sb.size] = sb
    codes = np.tile(np.arange(16, dtype=np.uint8)[:, None], (32, n_pad))              # [512, N]: row k -> q = k % 16
    zc = np.tile(np.arange(16, dtype=np.uint8)[:, None], (1, n_pad))                  # group g -> z = g
    scales = np.tile(s.view(np.float32)[None, :], (16, 1))
    g_idx = (np.arange(512) // 32).astype(np.int32)
    return o.pack_qweight(codes), o.pack_qzeros(zc), scales, g_idx, sb.size


def _scalar_table_of(W_bits, n):
    """[512, N] patterns of that layer -> [scale, q, z]."""
    return W_bits.reshape(16, 2, 16, -1)[:, 0, :, :n].transpose(2, 1, 0)


def test_generator_round_to_binary32_on_known_values():
    """The fixture generator's own rounding against values whose binary32 pattern is known by hand."""
    from fractions import Fraction
    gen = _load_generator()
    assert gen.rn32(Fraction(1)) == 0x3F800000 and gen.rn32(Fraction(-2)) == 0xC0000000
    assert gen.rn32(Fraction(1, 10)) == 0x3DCCCCCD and gen.rn32(Fraction(1, 3)) == 0x3EAAAAAB
    assert gen.rn32(1 + Fraction(1, 1 << 24)) == 0x3F800000            # tie -> even (down)
    assert gen.rn32(1 + Fraction(3, 1 << 24)) == 0x3F800002            # tie -> even (up)
    assert gen.rn32(2 - Fraction(1, 1 << 25)) == 0x40000000            # carries into the next binade
    assert gen.rn32(Fraction(1, 1 << 149)) == 0x00000001 and gen.rn32(Fraction(1, 1 << 150)) == 0   # subnormal, tie to 0
    assert gen.rn32(Fraction(3, 1 << 150)) == 0x00000002
    for u in (0x00000001, 0x007FFFFF, 0x00800000, 0x3FFFFFFF, 0xBF800001, 0x7B7FFFFF):
        assert gen.rn32(gen.float_bits_to_fraction(u)) == u


def test_dequant_f32_matches_golden_scalar_table_both_forms():
    qw, qz, scales, g_idx, n = _scalar_layer_f32()
    for fused, key in ((True, "scalar_fused"), (False, "scalar_separate")):
        got = _scalar_table_of(o.dequant_v2_f32(qw, qz, scales, g_idx, fused=fused).view(np.uint32), n)
        exp = GOLD32[key]
        same = (got == exp) | (((got | exp) & 0x7FFFFFFF) == 0)                            # +0 == -0
        assert same.all(), key


def test_dequant_f32_fused_and_separate_forms_are_distinguishable_and_within_one_ulp():
    f, s = GOLD32["scalar_fused"].astype(np.int64), GOLD32["scalar_separate"].astype(np.int64)
    typical = slice(0, 160)                                     # the GPTQ-magnitude scales
    differ = f[typical] != s[typical]
    assert 0.01 < differ.mean() < 0.6                           # a merged or split rounding in the oracle would show
    both_nonzero = ((f & 0x7FFFFFFF) != 0) & ((s & 0x7FFFFFFF) != 0) & ((f >> 31) == (s >> 31))
    # rounding the product first moves it by half a unit of ITS last place, which the difference can magnify
    # when it cancels; for same-sign neighbours the patterns are adjacent or a few steps apart
    gap = np.abs(f - s)[both_nonzero]
    assert np.median(gap[gap > 0]) == 1


def test_dequant_f32_matches_golden_act_order_layer():
    W = o.dequant_v2_f32(GOLD32["layer_qweight"], GOLD32["layer_qzeros"], GOLD32["layer_scales"], GOLD32["layer_g_idx"])
    assert np.array_equal(W.view(np.uint32), GOLD32["layer_W_bits"])
    # with fp16-representable scales and the fp16 flavour's operands the float result rounds to ... the exact value:
    # s*q - s*(z+1) needs at most 11 + 5 bits, so both float forms are exact there and equal (q - z - 1) * s
    lay = o.make_layer(128, 64, 32, act_order=True, seed=3)
    s32 = lay["scales"].astype(np.float32)
    for fused in (True, False):
        W32 = o.dequant_v2_f32(lay["qweight"], lay["qzeros"], s32, lay["g_idx"], fused=fused)
        q = o.unpack_qweight(lay["qweight"]).astype(np.float64)
        z = o.unpack_qzeros(lay["qzeros"]).astype(np.float64)[lay["g_idx"]]
        assert np.array_equal(W32.astype(np.float64), (q - z - 1.0) * s32[lay["g_idx"]].astype(np.float64))
