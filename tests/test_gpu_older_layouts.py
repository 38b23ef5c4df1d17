"""v1 (per-column fp16 scale / zero) and 2-bit v2 layers: dense dequantization on the GPU, bit-exact with
the oracle (quant_cuda_kernel.cu:1076-1097 and 1185-1211 of the reference), then a library GEMM
(matmul_utils_4bit.py:98-143); module forward / backward as Autograd4bitQuantLinear(is_v1_model=True / bits=2)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _v1_layer(oracle, K, N, seed):
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    scales = rng.uniform(0.005, 0.02, size=(N, 1)).astype(np.float16)
    zeros = (scales.astype(np.float32) * rng.integers(1, 17, size=(N, 1))).astype(np.float16)
    return oracle.pack_qweight(codes), scales, zeros


def _b2_layer(oracle, K, N, gs, seed, act_order=False):
    rng = np.random.default_rng(seed)
    G = K // gs
    codes = rng.integers(0, 4, size=(K, N), dtype=np.uint8)
    zc = rng.integers(0, 4, size=(G, N), dtype=np.uint8)
    scales = rng.uniform(0.01, 0.1, size=(G, N)).astype(np.float16)
    g_idx = (np.arange(K) // gs).astype(np.int32)
    if act_order:
        g_idx = g_idx[rng.permutation(K)].copy()
    return oracle.pack_qweight2(codes), oracle.pack_qzeros2(zc), scales, g_idx


@pytest.mark.parametrize("K,N", [(256, 128), (4096, 4096), (264, 64)])
def test_dequant_v1_bit_exact(oracle, K, N):
    from alpaca_lora_4bit_amd import quant_hip
    qw, s, z = _v1_layer(oracle, K, N, K + N)
    ref = oracle.dequant_v1(qw, s, z)
    got = quant_hip.dequant_v1(torch.from_numpy(qw).cuda(), torch.from_numpy(s).cuda(), torch.from_numpy(z).cuda())
    assert np.array_equal(got.cpu().numpy().view(np.uint16), ref.view(np.uint16))
    res = torch.empty((K, N), dtype=torch.float16, device="cuda")
    quant_hip.vecquant4recons_v1(torch.from_numpy(qw).cuda(), res, torch.from_numpy(s).cuda(), torch.from_numpy(z).cuda())
    assert torch.equal(res, got)


@pytest.mark.parametrize("K,N", [(4096, 4096), (512, 256), (1408, 192), (64, 64)])
@pytest.mark.parametrize("M", [1, 5, 16])
def test_gemv_v1(oracle, K, N, M):
    """Decode product of a v1 layer (the reference's vecquant4matmul_v1_faster): within 1e-2 of the fp32 product
    with the bit-exact dense W; accumulates into y on request; the pybind-style wrapper adds into `mul`."""
    from alpaca_lora_4bit_amd import quant_hip
    qw, s, z = _v1_layer(oracle, K, N, K + N + M)
    t = lambda a: torch.from_numpy(a).cuda()
    W = oracle.dequant_v1(qw, s, z).astype(np.float32)
    x = oracle.make_activations(M, K, seed=M)
    ref = x.astype(np.float32) @ W
    y = quant_hip.gemv_v1(t(x), t(qw), t(s), t(z))
    assert y.shape == (M, N) and y.dtype == torch.float16
    assert np.abs(y.float().cpu().numpy() - ref).max() <= 1e-2 * np.abs(ref).max()
    assert np.abs(y.float().cpu().numpy() - ref).max() <= 2e-3 * np.abs(ref).max()
    assert torch.equal(quant_hip.gemv_v1(t(x), t(qw), t(s), t(z)), y)              # reproducible
    base = torch.randn(M, N, device="cuda").half()
    acc = base.clone()
    quant_hip.gemv_v1(t(x), t(qw), t(s), t(z), out=acc, accumulate=True)
    assert torch.allclose(acc.float(), base.float() + y.float(), rtol=0, atol=2e-3 * float(np.abs(ref).max()) + 2e-3)
    mul = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    quant_hip.vecquant4matmul_v1_faster(t(x), t(qw), mul, t(s), t(z))
    assert torch.equal(mul, y)


@pytest.mark.parametrize("K,N,gs,act", [(256, 128, 128, False), (4096, 1024, 128, False), (512, 192, 64, True),
                                        (272, 64, 16, True)])
def test_dequant2_bit_exact(oracle, K, N, gs, act):
    from alpaca_lora_4bit_amd import quant_hip
    qw, qz, s, g = _b2_layer(oracle, K, N, gs, K + N, act)
    ref = oracle.dequant2_v2(qw, qz, s, g)
    t = lambda a: torch.from_numpy(a).cuda()
    got = quant_hip.dequant2(t(qw), t(qz), t(s), t(g), gs)
    assert np.array_equal(got.cpu().numpy().view(np.uint16), ref.view(np.uint16))
    if not act:
        assert torch.equal(quant_hip.dequant2(t(qw), t(qz), t(s), None, gs), got)


@pytest.mark.parametrize("rows", [1, 40])
def test_v1_module_forward_backward(oracle, rows):
    from alpaca_lora_4bit_amd.autograd_4bit import Autograd4bitQuantLinear
    K, N = 512, 256
    qw, s, z = _v1_layer(oracle, K, N, 3)
    m = Autograd4bitQuantLinear(K, N, is_v1_model=True).cuda()
    m.qweight, m.scales, m.zeros = torch.from_numpy(qw).cuda(), torch.from_numpy(s).cuda(), torch.from_numpy(z).cuda()
    m.bias = torch.zeros(N, dtype=torch.float16, device="cuda")
    W = oracle.dequant_v1(qw, s, z).astype(np.float32)
    x = oracle.make_activations(rows, K, seed=rows)
    dy = oracle.make_activations(rows, N, seed=rows + 1)
    xd = torch.from_numpy(x).cuda().requires_grad_(True)
    y = m(xd)
    y.backward(torch.from_numpy(dy).cuda())
    ref_y, ref_dx = x.astype(np.float32) @ W, dy.astype(np.float32) @ W.T
    assert np.abs(y.detach().float().cpu().numpy() - ref_y).max() <= 1e-2 * np.abs(ref_y).max()
    assert np.abs(xd.grad.float().cpu().numpy() - ref_dx).max() <= 1e-2 * np.abs(ref_dx).max()
    with torch.no_grad():                                   # no-grad dispatcher: the v1 GEMV for a few rows, else the same route
        y2 = m(torch.from_numpy(x).cuda())
    if rows > 8:
        assert torch.equal(y2, y.detach())
    else:
        assert np.abs(y2.float().cpu().numpy() - ref_y).max() <= 1e-2 * np.abs(ref_y).max()


def test_2bit_module_forward_backward(oracle):
    from alpaca_lora_4bit_amd.autograd_4bit import Autograd4bitQuantLinear
    K, N, gs, rows = 512, 256, 128, 33
    qw, qz, s, g = _b2_layer(oracle, K, N, gs, 9)
    m = Autograd4bitQuantLinear(K, N, groupsize=gs, bits=2).cuda()
    assert tuple(m.qweight.shape) == (K // 16, N) and tuple(m.qzeros.shape) == (K // gs, N // 16)
    t = lambda a: torch.from_numpy(a).cuda()
    m.qweight, m.qzeros, m.scales, m.g_idx = t(qw), t(qz), t(s), t(g)
    m.bias = torch.zeros(N, dtype=torch.float16, device="cuda")
    W = oracle.dequant2_v2(qw, qz, s, g).astype(np.float32)
    x = oracle.make_activations(rows, K, seed=1)
    dy = oracle.make_activations(rows, N, seed=2)
    xd = t(x).requires_grad_(True)
    y = m(xd)
    y.backward(t(dy))
    ref_y, ref_dx = x.astype(np.float32) @ W, dy.astype(np.float32) @ W.T
    assert np.abs(y.detach().float().cpu().numpy() - ref_y).max() <= 1e-2 * np.abs(ref_y).max()
    assert np.abs(xd.grad.float().cpu().numpy() - ref_dx).max() <= 1e-2 * np.abs(ref_dx).max()
