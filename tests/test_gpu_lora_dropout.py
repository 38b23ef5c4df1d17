"""Dropout in front of lora_A (the reference's default: --lora_dropout 0.05, arg_parser.py:48, applied at
models.py:63-66) inside the fused adapter kernels.  The mask is counter-based (a pure function of seed, row,
column; formula in include/q4_gptq.h), so every kernel regenerates it.  Checked here:
  * the mask the library writes out equals the numpy restatement of the documented formula, bit for bit, and has
    the statistics of a dropout mask;
  * q4_lora_down_f16, q4_lora_grad_f32 / _pair_f32, q4_gemm_bwd_dx_f16 with a dropout descriptor against float64
    products under that mask;
  * Linear4bitLt in training mode with p = 0.05 runs AutogradMatmul4bitLora and gives the oracle's y, dx, dA, dB
    for the same mask (1e-2 * max|ref|), including the full benchmark shape (2048 x 4096 -> 4096)."""
import numpy as np
import pytest
import torch

from conftest import rel_err, to_cuda_layer

pytestmark = pytest.mark.gpu
TOL = 1e-2


@pytest.mark.parametrize("M,C,seed,p", [(64, 256, 1, 0.05), (300, 4096, 2 ** 61 + 12345, 0.5), (7, 11008, 0xDEADBEEFCAFE, 0.1),
                                         (2048, 4096, 77, 0.05), (5, 64, 9, 0.0)])
def test_mask_matches_the_documented_formula(oracle, M, C, seed, p):
    from alpaca_lora_4bit_amd import quant_hip
    keep = quant_hip.dropout_keep_mask(M, C, seed, p).cpu().numpy()
    want, scale = oracle.dropout_keep_counter(M, C, seed, p)
    assert np.array_equal(keep, want)
    assert abs(quant_hip.dropout_scale(p) - scale) < 1e-6
    if M * C >= 1 << 20:
        n = M * C
        assert abs(keep.mean() - (1 - p)) < 4 * np.sqrt(p * (1 - p) / n) + 2e-5      # realized p is a multiple of 2^-15
        # neighbours along rows and along columns are uncorrelated
        assert abs(np.corrcoef(keep[:, :-1].ravel(), keep[:, 1:].ravel())[0, 1]) < 5e-3
        assert abs(np.corrcoef(keep[:-1].ravel(), keep[1:].ravel())[0, 1]) < 5e-3
    if p == 0.0:
        assert keep.all()


@pytest.mark.parametrize("M,C,R,wdtype", [(2048, 4096, 8, torch.float32), (37, 256, 16, torch.float16),
                                          (300, 11008, 64, torch.float32), (16, 4096, 3, torch.float32)])
def test_lora_down_with_dropout(oracle, M, C, R, wdtype):
    from alpaca_lora_4bit_amd import quant_hip
    rng = np.random.default_rng(M + C + R)
    x = rng.standard_normal((M, C)).astype(np.float16)
    w = (rng.standard_normal((R, C)) * 0.05).astype(np.float16)
    seed, p = 1234567 + M, 0.05
    keep, scale = oracle.dropout_keep_counter(M, C, seed, p)
    ref = (x.astype(np.float64) * keep * scale) @ w.astype(np.float64).T
    xd, wd = torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda().to(wdtype)
    for wv in (wd, wd.t().contiguous().t()):                       # lora_A layout and lora_B layout
        got = quant_hip.lora_down(xd, wv, dropout=(seed, p)).float().cpu().numpy()
        assert np.abs(got - ref).max() <= TOL * np.abs(ref).max() + 1e-6
    # another seed is another mask; p = 0 is the plain product
    other = quant_hip.lora_down(xd, wd, dropout=(seed + 1, p))
    assert not torch.equal(other, quant_hip.lora_down(xd, wd, dropout=(seed, p)))
    assert torch.equal(quant_hip.lora_down(xd, wd, dropout=(seed, 0.0)), quant_hip.lora_down(xd, wd))


@pytest.mark.parametrize("M,C,R", [(2048, 4096, 8), (2048, 4096, 16), (77, 64, 8), (1000, 520, 8)])
def test_lora_grad_with_dropout(oracle, M, C, R):
    from alpaca_lora_4bit_amd import quant_hip
    rng = np.random.default_rng(M + 3 * C + R)
    pm = (rng.standard_normal((M, R)) * 0.1).astype(np.float16)
    x = rng.standard_normal((M, C)).astype(np.float16)
    x2 = rng.standard_normal((M, 256)).astype(np.float16)
    seed, p, alpha = 99 + C, 0.05, 2.0
    keep, scale = oracle.dropout_keep_counter(M, C, seed, p)
    ref = alpha * (pm.astype(np.float64).T @ (x.astype(np.float64) * keep * scale))
    pd, xd, x2d = torch.from_numpy(pm).cuda(), torch.from_numpy(x).cuda(), torch.from_numpy(x2).cuda()
    got = quant_hip.lora_grad(pd, xd, alpha, dropout=(seed, p)).cpu().numpy()
    assert np.abs(got - ref).max() <= 1e-3 * np.abs(ref).max() + 1e-6
    # pair: the mask applies to the first problem only
    g1, g2 = quant_hip.lora_grad_pair(pd, xd, pd, x2d, alpha, dropout=(seed, p))
    assert np.abs(g1.cpu().numpy() - ref).max() <= 1e-3 * np.abs(ref).max() + 1e-6
    ref2 = alpha * (pm.astype(np.float64).T @ x2.astype(np.float64))
    assert np.abs(g2.cpu().numpy().T - ref2).max() <= 1e-3 * np.abs(ref2).max() + 1e-6


@pytest.mark.parametrize("M,K,N,r", [(256, 512, 384, 8), (2048, 4096, 4096, 8), (100, 256, 128, 16), (40, 1024, 256, 8)])
def test_gemm_bwd_dx_with_masked_adapter_term(oracle, M, K, N, r):
    """dx = dy @ W^T + mask/(1-p) * (s * dyb @ A): split reduction (few tiles), full tiles, 128-row tiles."""
    from alpaca_lora_4bit_amd import quant_hip
    layer = oracle.make_layer(K, N, 128, seed=K + N)
    t = to_cuda_layer(layer)
    A, _ = oracle.make_lora(K, N, r, seed=5)
    rng = np.random.default_rng(M)
    dy = oracle.make_activations(M, N, seed=61)
    dyb = (rng.standard_normal((M, r)) * 0.5).astype(np.float16)
    seed, p, s = 424242, 0.05, 2.0
    keep, scale = oracle.dropout_keep_counter(M, K, seed, p)
    W = oracle.dequant_v2(layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"]).astype(np.float64)
    ref = dy.astype(np.float64) @ W.T + keep * scale * (s * (dyb.astype(np.float64) @ A.astype(np.float64)))
    got = quant_hip.gemm_bwd_dx(torch.from_numpy(dy).cuda(), t["qweight"], t["qzeros"], t["scales"], None, 128,
                                dyb=torch.from_numpy(dyb).cuda(), lora_a=torch.from_numpy(A).cuda(), lora_scale=s,
                                dropout=(seed, p))
    assert rel_err(got.cpu().numpy(), ref) <= TOL
    # the adapter term alone (difference to the product without adapter) vanishes exactly where the mask drops
    base = quant_hip.gemm_bwd_dx(torch.from_numpy(dy).cuda(), t["qweight"], t["qzeros"], t["scales"], None, 128)
    diff = (got.float() - base.float()).cpu().numpy()
    term = s * scale * (dyb.astype(np.float64) @ A.astype(np.float64))
    # (both outputs are rounded to fp16, so their difference carries up to two roundings of the full-size value)
    assert np.abs(diff - term * keep).max() <= 2e-3 * max(np.abs(ref).max(), 1.0)
    assert np.abs(term[keep == 1]).max() > 20 * np.abs(diff[keep == 0]).max()


@pytest.mark.parametrize("act", [False, True])
@pytest.mark.parametrize("rows,K,N,r", [(2048, 4096, 4096, 8), (96, 256, 384, 16)])
def test_linear4bitlt_training_with_default_dropout_runs_the_fused_path(oracle, monkeypatch, rows, K, N, r, act):
    from alpaca_lora_4bit_amd import autograd_4bit, models
    layer = oracle.make_layer(K, N, 128, act_order=act, seed=23)
    A, B = oracle.make_lora(K, N, r, seed=23)
    m = models.Linear4bitLt("default", K, N, 128, False, r=r, lora_alpha=2 * r, lora_dropout=0.05).cuda()
    for k in ("qweight", "qzeros", "scales", "g_idx"):
        setattr(m, k, torch.from_numpy(layer[k]).cuda())
    m.bias = torch.zeros(N, dtype=torch.float16, device="cuda")
    m.lora_A["default"].weight.data = torch.from_numpy(A).cuda()
    m.lora_B["default"].weight.data = torch.from_numpy(B).cuda()
    m.train()
    calls = []
    real_apply = autograd_4bit.AutogradMatmul4bitLora.apply
    monkeypatch.setattr(autograd_4bit.AutogradMatmul4bitLora, "apply",
                        staticmethod(lambda *a: (calls.append(a[-2:]), real_apply(*a))[1]))
    x = oracle.make_activations(rows, K, seed=51)
    dy = oracle.make_activations(rows, N, seed=52)
    torch.manual_seed(2024)
    xt = torch.from_numpy(x).cuda().requires_grad_(True)
    with torch.amp.autocast(device_type="cuda"):
        y = m(xt)
    y.backward(torch.from_numpy(dy).cuda())
    assert len(calls) == 1 and calls[0][0] == 0.05                  # the fused Function ran, with the layer's p
    seed = calls[0][1]
    torch.manual_seed(2024)
    assert seed == int(torch.randint(0, 2 ** 62, (1,)).item())      # drawn from torch's generator: reproducible
    keep, scale = oracle.dropout_keep_counter(rows, K, seed, 0.05)
    W = oracle.dequant_v2(layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"]).astype(np.float64)
    yref = oracle.lora_forward(x, W, A, B, 2.0, keep=keep, drop_scale=scale)
    dxref, dAref, dBref = oracle.lora_backward(x, dy, W, A, B, 2.0, keep=keep, drop_scale=scale)
    assert rel_err(y.detach().cpu().numpy(), yref) <= TOL
    assert rel_err(xt.grad.cpu().numpy(), dxref) <= TOL
    assert rel_err(m.lora_A["default"].weight.grad.cpu().numpy(), dAref) <= TOL
    assert rel_err(m.lora_B["default"].weight.grad.cpu().numpy(), dBref) <= TOL
    # the mask matters: the no-dropout oracle is measurably different in the adapter gradient
    _, dA0, _ = oracle.lora_backward(x, dy, W, A, B, 2.0)
    assert rel_err(m.lora_A["default"].weight.grad.cpu().numpy(), dA0) > 2e-2
    # eval mode: no dropout, same Function
    m.eval()
    with torch.no_grad(), torch.amp.autocast(device_type="cuda"):
        y_eval = m(torch.from_numpy(x).cuda())
    assert rel_err(y_eval.cpu().numpy(), oracle.lora_forward(x, W, A, B, 2.0)) <= TOL
