"""Module-level parity: Autograd4bitQuantLinear / AutogradMatmul4bit / Linear4bitLt against
(i) the CPU oracle and (ii) torch autograd through a dense nn.Linear holding the oracle's W."""
import numpy as np
import pytest

from conftest import rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _fill(module, layer):
    import torch
    module.qweight = torch.from_numpy(layer["qweight"]).cuda()
    module.qzeros = torch.from_numpy(layer["qzeros"]).cuda()
    module.scales = torch.from_numpy(layer["scales"]).cuda()
    module.g_idx = torch.from_numpy(layer["g_idx"]).cuda()
    module.bias = torch.zeros(layer["N"], dtype=torch.float16, device="cuda")
    return module


@pytest.mark.parametrize("act", [False, True])
@pytest.mark.parametrize("shape", [(1, 1), (2, 4), (1, 16), (3, 40), (8, 256)])
def test_quant_linear_forward_both_modes(oracle, shape, act):
    """[batch, seq, K] inputs; no-grad (dispatcher) and grad mode (autograd Function) agree with
    the oracle; leading dimensions are preserved (autograd_4bit.py:192-208)."""
    import torch
    from alpaca_lora_4bit_amd.autograd_4bit import Autograd4bitQuantLinear
    K, N = 512, 384
    layer = oracle.make_layer(K, N, 128, act_order=act, seed=13)
    m = _fill(Autograd4bitQuantLinear(K, N, groupsize=128), layer)
    rng = np.random.default_rng(5)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float16)
    m.bias = torch.from_numpy(bias).cuda()
    x = oracle.make_activations(shape[0] * shape[1], K, seed=3).reshape(shape[0], shape[1], K)
    ref = oracle.matmul_recons(x.reshape(-1, K), layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    ref = (ref + bias.astype(np.float32)).reshape(shape[0], shape[1], N)
    xt = torch.from_numpy(x).cuda()
    with torch.no_grad():
        y0 = m(xt)
    y1 = m(xt.clone().requires_grad_(True))
    assert y0.shape == (shape[0], shape[1], N) and y0.dtype == torch.float16
    assert rel_err(y0.cpu().numpy(), ref) <= TOL
    assert rel_err(y1.detach().cpu().numpy(), ref) <= TOL
    m.disable_bias = True
    with torch.no_grad():
        y2 = m(xt)
    assert rel_err(y2.cpu().numpy(), ref - bias.astype(np.float32)) <= TOL


@pytest.mark.parametrize("rows", [4, 64])
def test_autograd_matches_dense_linear(oracle, rows):
    """dx from AutogradMatmul4bit.backward == dx of a dense fp32 nn.Linear built from W_ref;
    the six non-input gradients are None (autograd_4bit.py:54)."""
    import torch
    from alpaca_lora_4bit_amd import autograd_4bit
    K, N = 256, 384
    layer = oracle.make_layer(K, N, 128, seed=17)
    W = oracle.dequant_v2(layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    dense = torch.nn.Linear(K, N, bias=False).cuda()
    dense.weight.data = torch.from_numpy(W.astype(np.float32)).cuda().t().contiguous()
    x = torch.from_numpy(oracle.make_activations(rows, K, seed=1)).cuda()
    dy = torch.from_numpy(oracle.make_activations(rows, N, seed=2)).cuda()

    xq = x.clone().requires_grad_(True)
    t = {k: torch.from_numpy(layer[k]).cuda() for k in ("qweight", "qzeros", "scales", "g_idx")}
    y = autograd_4bit.AutogradMatmul4bit.apply(xq, t["qweight"], t["scales"], t["qzeros"], t["g_idx"], 4, 15)
    y.backward(dy)
    xd = x.float().clone().requires_grad_(True)
    yd = dense(xd)
    yd.backward(dy.float())
    assert rel_err(y.detach().cpu().numpy(), yd.detach().cpu().numpy()) <= TOL
    assert rel_err(xq.grad.cpu().numpy(), xd.grad.cpu().numpy()) <= TOL
    assert xq.grad.dtype == torch.float16


def test_autocast_casts_fp32_inputs(oracle):
    """Under autocast custom_fwd(cast_inputs=fp16) casts x and scales (autograd_4bit.py:35)."""
    import torch
    from alpaca_lora_4bit_amd.autograd_4bit import Autograd4bitQuantLinear
    K, N = 256, 128
    layer = oracle.make_layer(K, N, 128, seed=19)
    m = _fill(Autograd4bitQuantLinear(K, N, groupsize=128), layer)
    x = oracle.make_activations(32, K, seed=4)
    ref = oracle.matmul_recons(x, layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    xt = torch.from_numpy(x).cuda().float().requires_grad_(True)
    with torch.amp.autocast(device_type="cuda"):
        y = m(xt)
    assert y.dtype == torch.float16
    assert rel_err(y.detach().cpu().numpy(), ref) <= TOL
    y.float().sum().backward()
    assert xt.grad is not None and xt.grad.dtype == torch.float32


@pytest.mark.parametrize("act", [False, True])
@pytest.mark.parametrize("rows,K,N,r", [(2048, 4096, 4096, 8), (96, 256, 384, 16), (4, 256, 128, 8)])
def test_linear4bitlt_forward_backward(oracle, rows, K, N, r, act):
    """Linear4bitLt (fused path for rows > 16, reference composition otherwise) vs the closed-form
    oracle: y, dx, dA, dB.  Config 2 is the first parameter set."""
    import torch
    from alpaca_lora_4bit_amd import models
    layer = oracle.make_layer(K, N, 128, act_order=act, seed=23)
    A, B = oracle.make_lora(K, N, r, seed=23)
    m = models.Linear4bitLt("default", K, N, 128, False, r=r, lora_alpha=2 * r, lora_dropout=0.0).cuda()
    _fill(m, layer)
    m.lora_A["default"].weight.data = torch.from_numpy(A).cuda()
    m.lora_B["default"].weight.data = torch.from_numpy(B).cuda()
    assert m.scaling["default"] == 2.0
    x = oracle.make_activations(rows, K, seed=51)
    dy = oracle.make_activations(rows, N, seed=52)
    W = oracle.dequant_v2(layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"]).astype(np.float64)
    yref = oracle.lora_forward(x, W, A, B, 2.0)
    dxref, dAref, dBref = oracle.lora_backward(x, dy, W, A, B, 2.0)

    xt = torch.from_numpy(x).cuda().requires_grad_(True)
    with torch.amp.autocast(device_type="cuda"):
        y = m(xt)
    y.backward(torch.from_numpy(dy).cuda())
    assert y.dtype == torch.float16 and y.shape == (rows, N)
    assert rel_err(y.detach().cpu().numpy(), yref) <= TOL
    assert rel_err(xt.grad.cpu().numpy(), dxref) <= TOL
    gA, gB = m.lora_A["default"].weight.grad, m.lora_B["default"].weight.grad
    assert gA.dtype == torch.float32 and gB.dtype == torch.float32
    assert rel_err(gA.cpu().numpy(), dAref) <= TOL
    assert rel_err(gB.cpu().numpy(), dBref) <= TOL
    assert m.qweight.grad is None and m.scales.grad is None


def test_fused_and_unfused_lora_agree(oracle):
    import torch
    from alpaca_lora_4bit_amd import models
    K, N, r, rows = 512, 256, 8, 160
    layer = oracle.make_layer(K, N, 128, seed=29)
    A, B = oracle.make_lora(K, N, r, seed=29)
    m = models.Linear4bitLt("default", K, N, 128, False, r=r, lora_alpha=16).cuda()
    _fill(m, layer)
    m.lora_A["default"].weight.data = torch.from_numpy(A).cuda()
    m.lora_B["default"].weight.data = torch.from_numpy(B).cuda()
    x = torch.from_numpy(oracle.make_activations(rows, K, seed=6)).cuda()
    outs = []
    for fuse in (True, False):
        models.fuse_lora = fuse
        try:
            xt = x.clone().requires_grad_(True)
            with torch.amp.autocast(device_type="cuda"):
                y = m(xt)
            y.float().square().sum().backward()
            outs.append((y.detach().float().cpu().numpy(), xt.grad.float().cpu().numpy(),
                         m.lora_A["default"].weight.grad.clone().cpu().numpy(),
                         m.lora_B["default"].weight.grad.clone().cpu().numpy()))
            m.zero_grad()
        finally:
            models.fuse_lora = True
    for a, b in zip(*outs):
        assert rel_err(a, b) <= TOL


@pytest.mark.parametrize("rows", [1, 7, 16])
@pytest.mark.parametrize("wdtype", ["float32", "float16"])
def test_lora_layer_decode_path_matches_the_composition(oracle, rows, wdtype):
    """No-grad forward with a handful of rows: base GEMV + in-place rank-r update (three launches) gives the values
    of the reference's composition result + lora_B(lora_A(x)) * scaling (models.py:51-69), also after the adapter
    weights change and with a bias."""
    import torch
    from alpaca_lora_4bit_amd import models
    K, N, r = 512, 384, 8
    layer = oracle.make_layer(K, N, 128, seed=31)
    A, B = oracle.make_lora(K, N, r, seed=31)
    m = models.Linear4bitLt("default", K, N, 128, False, r=r, lora_alpha=16).cuda().eval()
    _fill(m, layer)
    dt = getattr(torch, wdtype)
    m.lora_A["default"].weight.data = torch.from_numpy(A).cuda().to(dt)
    m.lora_B["default"].weight.data = torch.from_numpy(B).cuda().to(dt)
    m.bias = torch.from_numpy((np.random.default_rng(5).standard_normal(N) * 0.1).astype(np.float16)).cuda()
    x = torch.from_numpy(oracle.make_activations(rows, K, seed=rows)).cuda().reshape(1, rows, K)
    W = oracle.dequant_v2(layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"]).astype(np.float64)

    def reference():
        a = m.lora_A["default"].weight.detach().double().cpu().numpy()
        b = m.lora_B["default"].weight.detach().double().cpu().numpy()
        xd = x.double().cpu().numpy().reshape(rows, K)
        return xd @ W + m.bias.double().cpu().numpy() + 2.0 * (xd @ a.T) @ b.T

    with torch.no_grad():
        y = m(x)
        assert y.shape == (1, rows, N) and y.dtype == torch.float16
        assert rel_err(y.reshape(rows, N).cpu().numpy(), reference()) <= TOL
        models.fuse_lora = False
        try:
            y_comp = m(x)
        finally:
            models.fuse_lora = True
        assert rel_err(y.cpu().numpy().reshape(rows, N), y_comp.float().cpu().numpy().reshape(rows, N)) <= 2e-3
        m.lora_B["default"].weight.mul_(3.0)                # in-place change: the cached fp16 copy must follow
        y2 = m(x)
        assert rel_err(y2.reshape(rows, N).cpu().numpy(), reference()) <= TOL
        assert not torch.equal(y2, y)


def test_fuse_quant_linears_matches_separate_layers(oracle):
    """gate/up (or q/k/v) concatenated along N: one launch, same numbers."""
    import torch
    from alpaca_lora_4bit_amd.autograd_4bit import Autograd4bitQuantLinear, fuse_quant_linears
    K = 512
    mods, refs = [], []
    x = oracle.make_activations(3, K, seed=9)
    for i, N in enumerate((256, 384)):
        layer = oracle.make_layer(K, N, 128, seed=40 + i)
        mods.append(_fill(Autograd4bitQuantLinear(K, N, groupsize=128), layer))
        refs.append(oracle.matmul_recons(x, layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"]))
    fused = fuse_quant_linears(mods)
    assert fused.out_features == 640 and fused.qweight.shape == (64, 640) and fused.qzeros.shape == (4, 80)
    xt = torch.from_numpy(x).cuda()
    with torch.no_grad():
        y = fused(xt)
        parts = torch.cat([m(xt) for m in mods], dim=-1)
    assert torch.equal(y, parts)
    assert rel_err(y.cpu().numpy(), np.concatenate(refs, axis=1)) <= TOL
    bad = Autograd4bitQuantLinear(K, 128, groupsize=64)
    with pytest.raises(ValueError):
        fuse_quant_linears([mods[0], bad])


def test_backend_switch_and_errors():
    from alpaca_lora_4bit_amd import autograd_4bit
    autograd_4bit.switch_backend_to("cuda")
    assert autograd_4bit.backend == "cuda"
    with pytest.raises(ValueError):
        autograd_4bit.switch_backend_to("triton")
    with pytest.raises(ValueError):
        autograd_4bit.switch_backend_to("metal")


@pytest.mark.parametrize("act", [False, True])
def test_dense_route_above_the_row_switch(oracle, act):
    """With matmul_utils_4bit.dense_switch_rows set, products above that many rows run as dense dequantization +
    library GEMM (the reference's recons scheme, matmul_utils_4bit.py:114-127; off by default): same values as the
    fused GEMM for the plain layer (no-grad and autograd, with bias) and for the LoRA layer (y, dx, dA, dB), and the
    fused kernels are not called."""
    import torch
    from alpaca_lora_4bit_amd import autograd_4bit, matmul_utils_4bit as mm4b, models, quant_hip
    K, N, r, rows = 256, 384, 8, 2304
    assert not mm4b.dense_switch_rows                      # default: the fused kernels at every size
    mm4b.dense_switch_rows = 2048
    layer = oracle.make_layer(K, N, 128, act_order=act, seed=31)
    A, B = oracle.make_lora(K, N, r, seed=31)
    x = oracle.make_activations(rows, K, seed=61)
    dy = oracle.make_activations(rows, N, seed=62)
    bias = (np.random.default_rng(7).standard_normal(N) * 0.1).astype(np.float16)
    W = oracle.dequant_v2(layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"]).astype(np.float64)

    fused_calls = []
    real_fwd, real_bwd = quant_hip.gemm_fwd, quant_hip.gemm_bwd_dx
    quant_hip.gemm_fwd = lambda *a, **k: (fused_calls.append("fwd"), real_fwd(*a, **k))[1]
    quant_hip.gemm_bwd_dx = lambda *a, **k: (fused_calls.append("bwd"), real_bwd(*a, **k))[1]
    try:
        plain = _fill(autograd_4bit.Autograd4bitQuantLinear(K, N, groupsize=128), layer)
        plain.bias = torch.from_numpy(bias).cuda()
        yref = x.astype(np.float64) @ W + bias.astype(np.float64)
        xt = torch.from_numpy(x).cuda()
        with torch.no_grad():
            assert rel_err(plain(xt).cpu().numpy(), yref) <= TOL
        xg = xt.clone().requires_grad_(True)
        y = plain(xg)
        y.backward(torch.from_numpy(dy).cuda())
        assert rel_err(y.detach().cpu().numpy(), yref) <= TOL
        assert rel_err(xg.grad.cpu().numpy(), dy.astype(np.float64) @ W.T) <= TOL

        m = models.Linear4bitLt("default", K, N, 128, False, r=r, lora_alpha=2 * r, lora_dropout=0.0).cuda()
        _fill(m, layer)
        m.bias = torch.from_numpy(bias).cuda()
        m.lora_A["default"].weight.data = torch.from_numpy(A).cuda()
        m.lora_B["default"].weight.data = torch.from_numpy(B).cuda()
        yl = oracle.lora_forward(x, W, A, B, 2.0) + bias.astype(np.float64)
        dxl, dAl, dBl = oracle.lora_backward(x, dy, W, A, B, 2.0)
        xg = xt.clone().requires_grad_(True)
        with torch.amp.autocast(device_type="cuda"):
            y = m(xg)
        y.backward(torch.from_numpy(dy).cuda())
        assert y.dtype == torch.float16 and y.shape == (rows, N)
        assert rel_err(y.detach().cpu().numpy(), yl) <= TOL
        assert rel_err(xg.grad.cpu().numpy(), dxl) <= TOL
        assert rel_err(m.lora_A["default"].weight.grad.cpu().numpy(), dAl) <= TOL
        assert rel_err(m.lora_B["default"].weight.grad.cpu().numpy(), dBl) <= TOL
        assert fused_calls == []

        # one row fewer than the switch: the fused kernels again, same numbers
        mm4b.dense_switch_rows = rows
        try:
            with torch.no_grad():
                assert rel_err(plain(xt).cpu().numpy(), yref) <= TOL
        finally:
            mm4b.dense_switch_rows = 2048
        assert fused_calls == ["fwd"]
    finally:
        mm4b.dense_switch_rows = None
        quant_hip.gemm_fwd, quant_hip.gemm_bwd_dx = real_fwd, real_bwd


@pytest.mark.parametrize("shape", [(0,), (2, 0), (0, 3)])
def test_empty_batches(oracle, shape):
    """Inputs without rows ([0, K], [2, 0, K], [0, 3, K]) give outputs without rows, in both modes, and zero
    adapter gradients; nothing is launched."""
    import torch
    from alpaca_lora_4bit_amd import autograd_4bit, models
    K, N, r = 256, 384, 8
    layer = oracle.make_layer(K, N, 128, seed=37)
    plain = _fill(autograd_4bit.Autograd4bitQuantLinear(K, N, groupsize=128), layer)
    plain.bias = torch.ones(N, dtype=torch.float16, device="cuda")
    lora = models.Linear4bitLt("default", K, N, 128, False, r=r, lora_alpha=16, lora_dropout=0.0).cuda()
    _fill(lora, layer)
    x = torch.zeros(shape + (K,), dtype=torch.float16, device="cuda")
    for m in (plain, lora):
        with torch.no_grad():
            y = m(x)
        assert y.shape == shape + (N,) and y.dtype == torch.float16
        xg = x.clone().requires_grad_(True)
        with torch.amp.autocast(device_type="cuda"):
            y = m(xg)
        assert y.shape == shape + (N,)
        y.sum().backward()
        assert xg.grad is not None and xg.grad.shape == x.shape
    for w in (lora.lora_A["default"].weight, lora.lora_B["default"].weight):
        assert w.grad is not None and float(w.grad.abs().max()) == 0.0


def test_layers_outside_the_tiled_kernels_take_the_dense_route(oracle):
    """in / out features that are not multiples of 128 (here 160 -> 192): above 16 rows the tiled kernels do not
    apply, the layer then runs dense dequantization + a library GEMM, forward and backward, like every layer of the
    reference (matmul_utils_4bit.py:114-127); up to 16 rows it takes the GEMV."""
    import torch
    from alpaca_lora_4bit_amd import models
    from alpaca_lora_4bit_amd.autograd_4bit import Autograd4bitQuantLinear
    K, N = 160, 192
    layer = oracle.make_layer(K, N, 32, seed=31)
    m = _fill(Autograd4bitQuantLinear(K, N, groupsize=32), layer)
    for rows in (1, 16, 17, 200):
        x = oracle.make_activations(rows, K, seed=rows)
        dy = oracle.make_activations(rows, N, seed=rows + 1)
        ref = oracle.matmul_recons(x, layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
        refx = oracle.matmul_recons_t(dy, layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
        xt = torch.from_numpy(x).cuda().requires_grad_(True)
        y = m(xt)
        y.backward(torch.from_numpy(dy).cuda())
        assert rel_err(y.detach().cpu().numpy(), ref) <= TOL
        assert rel_err(xt.grad.cpu().numpy(), refx) <= TOL
        with torch.no_grad():
            assert rel_err(m(torch.from_numpy(x).cuda()).cpu().numpy(), ref) <= TOL
    # with an adapter: the reference composition on top of the same route
    A, B = oracle.make_lora(K, N, 8, seed=3)
    lt = models.Linear4bitLt("default", K, N, 32, False, r=8, lora_alpha=16).cuda()
    _fill(lt, layer)
    lt.lora_A["default"].weight.data = torch.from_numpy(A).cuda()
    lt.lora_B["default"].weight.data = torch.from_numpy(B).cuda()
    x = oracle.make_activations(64, K, seed=9)
    W = oracle.dequant_v2(layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"]).astype(np.float64)
    with torch.amp.autocast(device_type="cuda"):
        y = lt(torch.from_numpy(x).cuda())
    assert rel_err(y.detach().float().cpu().numpy(), oracle.lora_forward(x, W, A, B, 2.0)) <= TOL


def test_decode_with_adapter_takes_a_strided_last_token_view(oracle):
    """h[:, -1:, :] of a batch is not contiguous: the short adapter path must accept it."""
    import torch
    from alpaca_lora_4bit_amd import models
    K, N, r = 256, 128, 8
    layer = oracle.make_layer(K, N, 128, seed=37)
    A, B = oracle.make_lora(K, N, r, seed=37)
    m = models.Linear4bitLt("default", K, N, 128, False, r=r, lora_alpha=16).cuda().eval()
    _fill(m, layer)
    m.lora_A["default"].weight.data = torch.from_numpy(A).cuda()
    m.lora_B["default"].weight.data = torch.from_numpy(B).cuda()
    h = torch.from_numpy(oracle.make_activations(3 * 5, K, seed=6)).cuda().view(3, 5, K)
    last = h[:, -1:, :]
    assert not last.is_contiguous()
    with torch.no_grad():
        y = m(last)
    W = oracle.dequant_v2(layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"]).astype(np.float64)
    ref = oracle.lora_forward(last.reshape(3, K).cpu().numpy(), W, A, B, 2.0)
    assert y.shape == (3, 1, N) and rel_err(y.reshape(3, N).cpu().numpy(), ref) <= TOL
