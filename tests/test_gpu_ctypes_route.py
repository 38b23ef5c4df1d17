"""quant_hip has two launch routes per operator: the compiled binding (_q4_host) and, for a tree where only the
library was built, ctypes.  The GPU suite otherwise runs the first; here every operator also runs with the binding
switched off.  Same C ABI and same kernels underneath, so the two routes must agree bit for bit; one of them is also
held to the oracle."""
import numpy as np
import pytest

from conftest import rel_err, to_cuda_layer

pytestmark = pytest.mark.gpu


@pytest.fixture
def routes(monkeypatch):
    from alpaca_lora_4bit_amd import quant_hip
    host = quant_hip._host
    assert host is not None, "the compiled host binding must be present in the GPU test tree"

    def both(fn):
        with_host = fn()
        monkeypatch.setattr(quant_hip, "_host", None)
        try:
            without = fn()
        finally:
            monkeypatch.setattr(quant_hip, "_host", host)
        return with_host, without
    return both


def _same(a, b):
    import torch
    if isinstance(a, (tuple, list)):
        return len(a) == len(b) and all(_same(x, y) for x, y in zip(a, b))
    return a.shape == b.shape and a.dtype == b.dtype and torch.equal(a, b)


@pytest.mark.parametrize("act_order", [False, True])
def test_every_operator_through_ctypes_matches_the_compiled_binding(oracle, routes, act_order):
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    K, N, gs, r = 1024, 768, 128, 8
    layer = oracle.make_layer(K, N, gs, act_order=act_order, seed=31)
    t = to_cuda_layer(layer)
    lay = (t["qweight"], t["qzeros"], t["scales"], t["g_idx"], gs)
    Wref = oracle.dequant_v2(layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    A, B = oracle.make_lora(K, N, r, seed=3)
    At, Bt = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    bias = torch.randn(N, device="cuda").half()

    a, b = routes(lambda: quant_hip.dequant(*lay))
    assert _same(a, b) and np.array_equal(a.cpu().numpy().view(np.uint16), Wref.view(np.uint16))

    for M in (1, 3, 16):
        xh = oracle.make_activations(M, K, seed=M)
        x = torch.from_numpy(xh).cuda()
        a, b = routes(lambda: quant_hip.gemv(x, *lay, out_shape=(1, M, N)))
        assert _same(a, b) and a.shape == (1, M, N)
        assert rel_err(a.reshape(M, N).cpu().numpy(), xh.astype(np.float64) @ Wref.astype(np.float64)) <= 1e-2
        base = torch.randn(M, N, device="cuda").half()
        a, b = routes(lambda: quant_hip.gemv(x, *lay, out=base.clone(), accumulate=True))
        assert _same(a, b)
    if not act_order:
        other = to_cuda_layer(oracle.make_layer(K, 256, gs, seed=32))
        x = torch.from_numpy(oracle.make_activations(2, K, seed=7)).cuda()
        a, b = routes(lambda: quant_hip.gemv_grouped(x, [lay[:3], (other["qweight"], other["qzeros"], other["scales"])], gs))
        assert _same(a, b) and a[0].shape == (2, N) and a[1].shape == (2, 256)

    for M in (40, 300):
        xh, dyh = oracle.make_activations(M, K, seed=M), oracle.make_activations(M, N, seed=M + 1)
        x, dy = torch.from_numpy(xh).cuda(), torch.from_numpy(dyh).cuda()
        xa, xa2 = routes(lambda: quant_hip.lora_down(x, At))
        dyb, dyb2 = routes(lambda: quant_hip.lora_down(dy, Bt.t()))
        assert _same(xa, xa2) and _same(dyb, dyb2)
        a, b = routes(lambda: quant_hip.gemm_fwd(x, *lay, bias=bias, xa=xa, lora_bt=Bt.t(), lora_scale=2.0))
        assert _same(a, b)
        ref = oracle.lora_forward(xh, Wref, A, B, 2.0) + bias.float().cpu().numpy()
        assert rel_err(a.cpu().numpy(), ref) <= 1e-2
        a, b = routes(lambda: quant_hip.gemm_fwd(x, *lay))
        assert _same(a, b)
        a, b = routes(lambda: quant_hip.gemm_bwd_dx(dy, *lay, dyb=dyb, lora_a=At, lora_scale=2.0))
        assert _same(a, b)
        dxref = oracle.lora_backward(xh, dyh, Wref, A, B, 2.0)[0]
        assert rel_err(a.cpu().numpy(), dxref) <= 1e-2
        a, b = routes(lambda: quant_hip.gemm_bwd_dx(dy, *lay, dyb=dyb, lora_a=At, lora_scale=2.0, dropout=(1234, 0.05)))
        assert _same(a, b)
        a, b = routes(lambda: quant_hip.lora_grad_pair(dyb, x, xa, dy, 2.0))
        assert _same(a, b)
        a, b = routes(lambda: quant_hip.lora_grad_pair(dyb, x, xa, dy, 2.0, dropout=(99, 0.05)))
        assert _same(a, b)
    assert quant_hip.workspaces_are_zero()
