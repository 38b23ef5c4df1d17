"""Parity of the rank-R adapter kernels (q4_lora_down_f16, q4_lora_grad_f32) with the numpy oracle's
adapter products (oracle/q4_oracle.py: lora_forward / lora_backward follow models.py:58-66 of the
reference and torch autograd over its two adapter Linears).

Tolerance: 1e-2 * max|ref| as for every matmul of this path; the fp32 gradients are additionally checked
to 1e-3 relative since they accumulate in fp32 / exact fixed point from the same fp16 inputs."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _rand16(rng, *shape, scale=1.0):
    return (rng.standard_normal(shape) * scale).astype(np.float16)


@pytest.mark.parametrize("M,C,R,wdtype", [
    (2048, 4096, 8, torch.float32), (2048, 4096, 8, torch.float16), (37, 256, 16, torch.float32),
    (1, 64, 8, torch.float16), (300, 11008, 64, torch.float32), (129, 1024, 24, torch.float16),
    (16, 4096, 3, torch.float32),
])
def test_lora_down_both_layouts(M, C, R, wdtype):
    from alpaca_lora_4bit_amd import quant_hip
    rng = np.random.default_rng(M * 7 + C + R)
    x = _rand16(rng, M, C)
    w = _rand16(rng, R, C, scale=0.05)
    ref = x.astype(np.float32) @ w.astype(np.float32).T
    xd = torch.from_numpy(x).cuda()
    wd = torch.from_numpy(w).cuda().to(wdtype)
    tol = 1e-2 * np.abs(ref).max() + 1e-6
    got = quant_hip.lora_down(xd, wd).float().cpu().numpy()                     # lora_A layout [R, C]
    assert np.abs(got - ref).max() <= tol
    wt = wd.t().contiguous()                                                   # lora_B layout [C, R], viewed as [R, C]
    got_t = quant_hip.lora_down(xd, wt.t()).float().cpu().numpy()
    assert np.abs(got_t - ref).max() <= tol
    assert np.array_equal(got, got_t)                                           # same arithmetic either way
    big = torch.zeros((R, C + 3), dtype=wdtype, device="cuda")                 # odd row pitch, unaligned start
    big[:, 1:C + 1] = wd
    got_v = quant_hip.lora_down(xd, big[:, 1:C + 1]).float().cpu().numpy()
    assert np.array_equal(got, got_v)


@pytest.mark.parametrize("M,C,R", [(2048, 4096, 8), (2048, 11008, 8), (2048, 4096, 16), (77, 64, 8),
                                   (1, 8, 16), (1000, 520, 8), (5000, 128, 16), (513, 4096, 4), (300, 264, 2),
                                   (1024, 4096, 32), (129, 136, 24), (40000, 128, 12)])
def test_lora_grad_matches_fp32_product(M, C, R):
    from alpaca_lora_4bit_amd import quant_hip
    rng = np.random.default_rng(M + C * 3 + R)
    p = _rand16(rng, M, R, scale=0.1)
    x = _rand16(rng, M, C)
    alpha = 2.0
    ref = alpha * (p.astype(np.float64).T @ x.astype(np.float64))
    pd, xd = torch.from_numpy(p).cuda(), torch.from_numpy(x).cuda()
    got = quant_hip.lora_grad(pd, xd, alpha)
    got_t = quant_hip.lora_grad(pd, xd, alpha, transposed=True)
    assert got.shape == (R, C) and got_t.shape == (C, R) and got.dtype == torch.float32
    g = got.cpu().numpy()
    assert np.abs(g - ref).max() <= 1e-3 * np.abs(ref).max() + 1e-6
    assert torch.equal(got, got_t.t())                                          # strided store, same sums
    # reproducible: the cross-workgroup sum is order-independent
    again = quant_hip.lora_grad(pd, xd, alpha)
    assert torch.equal(got, again)


def test_lora_grad_does_not_disturb_gemv_workspace(oracle):
    """The gradient's partial sums live in their own scratch: a GEMV (whose split-K workspace must stay
    zero between calls) gives the same result before and after."""
    from alpaca_lora_4bit_amd import quant_hip
    rng = np.random.default_rng(3)
    layer = oracle.make_layer(4096, 256, 128, seed=2)
    t = lambda a: torch.from_numpy(a).cuda()
    q, z, sc = t(layer["qweight"]), t(layer["qzeros"]), t(layer["scales"])
    x = t(oracle.make_activations(1, 4096, seed=9))
    y0 = quant_hip.gemv(x, q, z, sc, None, 128).clone()
    pd = t(_rand16(rng, 2048, 8))
    xd = t(_rand16(rng, 2048, 4096))
    quant_hip.lora_grad(pd, xd, 1.0)
    y1 = quant_hip.gemv(x, q, z, sc, None, 128)
    assert torch.equal(y0, y1)
    assert quant_hip.workspaces_are_zero()


def test_fused_lora_function_against_oracle_fp32_adapters(oracle):
    """Whole fused layer with fp32 adapter parameters (the usual PEFT state): y, dx, dA, dB against
    the oracle's float64 lora_forward / lora_backward on the fp16-rounded adapter values."""
    from alpaca_lora_4bit_amd.autograd_4bit import AutogradMatmul4bitLora
    K, N, M, r, gs = 512, 384, 200, 8, 128
    layer = oracle.make_layer(K, N, gs, seed=11)
    x = oracle.make_activations(M, K, seed=5)
    dy = oracle.make_activations(M, N, seed=6)
    A, B = oracle.make_lora(K, N, r, seed=7)
    B = (B * 10).astype(np.float32)                      # a trained-looking B so that every term matters
    scaling = 2.0
    W = oracle.dequant_v2(layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    A16, B16 = A.astype(np.float16), B.astype(np.float16)
    y_ref = oracle.lora_forward(x, W, A16, B16, scaling)
    dx_ref, dA_ref, dB_ref = oracle.lora_backward(x, dy, W, A16, B16, scaling)

    t = lambda a: torch.from_numpy(a).cuda()
    xd = t(x).requires_grad_(True)
    Ad = t(A).requires_grad_(True)
    Bd = t(B).requires_grad_(True)
    y = AutogradMatmul4bitLora.apply(xd, t(layer["qweight"]), t(layer["scales"]), t(layer["qzeros"]), None, None,
                                     Ad, Bd, scaling, gs)
    y.backward(t(dy))
    for got, ref in ((y, y_ref), (xd.grad, dx_ref), (Ad.grad, dA_ref), (Bd.grad, dB_ref)):
        g = got.detach().float().cpu().numpy()
        assert g.shape == ref.shape
        assert np.abs(g - ref).max() <= 1e-2 * np.abs(ref).max()
    assert Ad.grad.dtype == torch.float32 and Bd.grad.dtype == torch.float32


@pytest.mark.parametrize("M,C1,C2,R", [(2048, 4096, 4096, 8), (300, 1408, 512, 16), (50, 512, 11008, 8), (1000, 11008, 4096, 16),
                                       (700, 4096, 1024, 32), (2048, 128, 4096, 6)])
def test_lora_grad_pair_equals_the_two_single_launches(M, C1, C2, R):
    """Both gradients in one launch (different column counts, hence different grids and split counts) give the
    bits of the two separate launches."""
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    g = torch.Generator().manual_seed(M + C1 + R)
    p1 = torch.randn(M, R, generator=g).half().cuda()
    p2 = torch.randn(M, R, generator=g).half().cuda()
    in1 = torch.randn(M, C1, generator=g).half().cuda()
    in2 = torch.randn(M, C2, generator=g).half().cuda()
    want1 = quant_hip.lora_grad(p1, in1, 2.0)
    want2 = quant_hip.lora_grad(p2, in2, 2.0, transposed=True)
    got1, got2 = quant_hip.lora_grad_pair(p1, in1, p2, in2, 2.0)
    assert got1.shape == (R, C1) and got2.shape == (C2, R)
    assert torch.equal(got1, want1) and torch.equal(got2, want2)
    ref1 = 2.0 * p1.float().t() @ in1.float()
    assert float((got1 - ref1).abs().max() / ref1.abs().max()) <= 1e-3
