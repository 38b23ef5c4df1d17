"""Grouped GEMMs (q4_gemm_grouped_fwd_f16 / q4_gemm_grouped_bwd_dx_f16: q|k|v or gate|up of a block in one launch on the
layers' own tensors) against the CPU oracle and against the per-layer entry points.  Tolerance 1e-2 * max|ref|."""
import numpy as np
import pytest

from conftest import rel_err, to_cuda_layer

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _t(a):
    import torch
    return torch.from_numpy(a).cuda()


@pytest.mark.parametrize("M,K,Ns,gs,lora", [
    (1024, 4096, (4096, 4096, 4096), 128, (8, 0, 8)),          # q|k|v of config 4: 192 wide tiles, adapters on q and v
    (1024, 4096, (11008, 11008), 128, (0, 0)),                 # gate|up of config 4
    (600, 1024, (4096, 2048, 1024, 2048), 256, (16, 8, 0, 0)),  # four layers, ragged rows, narrow tiles, two shares per layer
    (2048, 512, (4096, 4096), 64, (0, 8)),                     # groups of 64 rows
])
def test_grouped_forward_and_grad_input(oracle, M, K, Ns, gs, lora):
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    assert quant_hip.gemm_grouped_applicable(True, M, K, Ns) and quant_hip.gemm_grouped_applicable(False, M, K, Ns)
    layers = [oracle.make_layer(K, N, gs, seed=K + N + i) for i, N in enumerate(Ns)]
    ts = [to_cuda_layer(l) for l in layers]
    xh = oracle.make_activations(M, K, seed=M)
    x = _t(xh)
    rng = np.random.default_rng(M + K)
    biases, As, Bs, xas = [], [], [], []
    for i, (N, r) in enumerate(zip(Ns, lora)):
        biases.append(torch.randn(N, device="cuda").half() if i % 2 == 0 else None)
        if r:
            A, B = oracle.make_lora(K, N, r, seed=i + 1)
            As.append(_t(A)); Bs.append(_t(B))
            xas.append(quant_hip.lora_down(x, As[-1]))
        else:
            As.append(None); Bs.append(None); xas.append(None)
    fwd_layers = [(t["qweight"], t["qzeros"], t["scales"], b, xa, None if B is None else B.t(), 2.0)
                  for t, b, xa, B in zip(ts, biases, xas, Bs)]
    ys = quant_hip.gemm_grouped_fwd(x, fwd_layers, gs)
    ys2 = quant_hip.gemm_grouped_fwd(x, fwd_layers, gs)
    rows = np.array([0, 1, M // 2, M - 1])
    for i, (lay, t, y) in enumerate(zip(layers, ts, ys)):
        assert y.shape == (M, Ns[i]) and torch.equal(y, ys2[i])
        single = quant_hip.gemm_fwd(x, t["qweight"], t["qzeros"], t["scales"], None, gs, bias=biases[i], xa=xas[i],
                                    lora_bt=None if Bs[i] is None else Bs[i].t(), lora_scale=2.0)
        assert float((y.float() - single.float()).abs().max() / single.float().abs().max()) <= 2e-3
        ref = oracle.matmul_recons(xh[rows], lay["qweight"], lay["qzeros"], lay["scales"], lay["g_idx"])
        if biases[i] is not None:
            ref = ref + biases[i].float().cpu().numpy()
        if lora[i]:
            ref = ref + 2.0 * (xas[i].float().cpu().numpy()[rows].astype(np.float64) @ Bs[i].half().float().cpu().numpy().astype(np.float64).T)
        assert rel_err(y.cpu().numpy()[rows], ref) <= 2e-3

    dyhs = [oracle.make_activations(M, N, seed=M + 7 + i) for i, N in enumerate(Ns)]
    dys = [_t(d) for d in dyhs]
    dybs = [None if B is None else quant_hip.lora_down(dy, B.t()) for dy, B in zip(dys, Bs)]
    for drops in ([None] * len(Ns), [(77 + i, 0.1) if lora[i] else None for i in range(len(Ns))]):
        bwd_layers = [(t["qweight"], t["qzeros"], t["scales"], dyb, A, 2.0, dr) for t, dyb, A, dr in zip(ts, dybs, As, drops)]
        dx = quant_hip.gemm_grouped_bwd_dx(dys, bwd_layers, gs)
        assert dx.shape == (M, K) and torch.equal(dx, quant_hip.gemm_grouped_bwd_dx(dys, bwd_layers, gs))
        want = torch.zeros(M, K, device="cuda")
        for t, dy, dyb, A, dr in zip(ts, dys, dybs, As, drops):
            want += quant_hip.gemm_bwd_dx(dy, t["qweight"], t["qzeros"], t["scales"], None, gs, dyb=dyb, lora_a=A, lora_scale=2.0,
                                          dropout=dr).float()
        assert float((dx.float() - want).abs().max() / want.abs().max()) <= 2e-3
        if drops[0] is None and not any(drops):
            ref = np.zeros((len(rows), K))
            for lay, dyh, dyb, A in zip(layers, dyhs, dybs, As):
                ref += oracle.matmul_recons_t(dyh[rows], lay["qweight"], lay["qzeros"], lay["scales"], lay["g_idx"])
                if A is not None:
                    ref += 2.0 * (dyb.float().cpu().numpy()[rows].astype(np.float64) @ A.half().float().cpu().numpy().astype(np.float64))
            assert rel_err(dx.cpu().numpy()[rows], ref) <= 2e-3


def test_grouped_gemm_refuses_what_it_does_not_take(oracle):
    import ctypes
    import torch
    from alpaca_lora_4bit_amd import _lib, quant_hip
    assert not quant_hip.gemm_grouped_applicable(True, 128, 4096, (4096, 4096, 4096))      # 128 rows: the per-layer kernels
    assert not quant_hip.gemm_grouped_applicable(True, 1024, 4096, (4096,))                # one layer is not a group
    assert not quant_hip.gemm_grouped_applicable(True, 256, 1024, (128, 128))              # too few tiles for a launch
    assert not quant_hip.gemm_grouped_applicable(False, 1024, 4096 + 64, (4096, 4096))
    L = _lib.lib()
    lay = to_cuda_layer(oracle.make_layer(256, 128, 128, seed=1))
    x = torch.zeros(256, 256, device="cuda", dtype=torch.float16)
    y = torch.zeros(256, 128, device="cuda", dtype=torch.float16)
    desc = (_lib.GemmLayer * 2)()
    for d in desc:
        d.act, d.qweight, d.qzeros, d.scales, d.out, d.N = (x.data_ptr(), lay["qweight"].data_ptr(), lay["qzeros"].data_ptr(),
                                                            lay["scales"].data_ptr(), y.data_ptr(), 128)
    assert L.q4_gemm_grouped_fwd_f16(desc, 2, 128, 256, 256, None) == -2                   # not enough tiles
    assert L.q4_gemm_grouped_fwd_f16(None, 2, 128, 256, 256, None) == -1
    assert L.q4_gemm_grouped_bwd_dx_f16(desc, 2, 128, None, 256, 256, None, 0, None) == -1


class _Block:
    """Stands for an attention block: three projections of one input, two of them with LoRA adapters."""

    def __new__(cls, oracle, K, N, gs, dropout, seed):
        import torch
        import torch.nn as nn
        from alpaca_lora_4bit_amd import autograd_4bit as ag, models

        class Block(nn.Module):
            def __init__(self):
                super().__init__()
                for i, name in enumerate(("q_proj", "k_proj", "v_proj")):
                    lay = oracle.make_layer(K, N, gs, seed=seed + i)
                    if name == "k_proj":
                        m = ag.Autograd4bitQuantLinear(K, N, groupsize=gs)
                    else:
                        m = models.Linear4bitLt("default", K, N, gs, False, r=8, lora_alpha=16, lora_dropout=dropout)
                        A, B = oracle.make_lora(K, N, 8, seed=seed + 10 + i)
                        m.lora_A["default"].weight.data = torch.from_numpy(A)
                        m.lora_B["default"].weight.data = torch.from_numpy(B)
                    m.qweight.data = torch.from_numpy(lay["qweight"])
                    m.qzeros.data = torch.from_numpy(lay["qzeros"])
                    m.scales = torch.from_numpy(lay["scales"])
                    m.g_idx.data = torch.from_numpy(lay["g_idx"])
                    m.bias = torch.zeros(N, dtype=torch.float16) if name != "v_proj" else (torch.arange(N) % 7 - 3).half() * 0.25
                    setattr(self, name, m)

            def forward(self, x):
                return self.q_proj(x), self.k_proj(x), self.v_proj(x)
        return Block().cuda()


@pytest.mark.parametrize("dropout", [0.0, 0.1])
def test_grouped_block_matches_the_ungrouped_block_forward_and_gradients(oracle, dropout, monkeypatch):
    """make_quant_attn on a block above the decode sizes: q|k|v (LoRA on q and v, a bias on v) run as ONE grouped
    forward launch and, in backward, ONE grouped grad-input launch.  Outputs, grad_input and adapter gradients
    against the same block ungrouped (whose layers are held to the oracle in test_gpu_autograd.py); with adapter
    dropout both draw their mask seeds in the same order, so the masks are the same."""
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    from alpaca_lora_4bit_amd.model_attn_mlp_patch import make_quant_attn, ungroup
    K, N, gs, M = 1024, 4096, 128, 512
    grouped, plain = _Block(oracle, K, N, gs, dropout, 40), _Block(oracle, K, N, gs, dropout, 40)
    assert make_quant_attn(grouped) == 1
    grouped.train(); plain.train()
    calls = {"fwd": 0, "bwd": 0}
    for name, key in (("gemm_grouped_fwd", "fwd"), ("gemm_grouped_bwd_dx", "bwd")):
        real = getattr(quant_hip, name)
        monkeypatch.setattr(quant_hip, name, (lambda real, key: lambda *a, **k: (calls.__setitem__(key, calls[key] + 1), real(*a, **k))[1])(real, key))
    xh = oracle.make_activations(M, K, seed=3)
    gys = [_t(oracle.make_activations(M, N, seed=4 + i)).view(2, M // 2, N) for i in range(3)]
    results = []
    for block in (grouped, plain):
        torch.manual_seed(1234)
        x = _t(xh).view(2, M // 2, K).requires_grad_(True)
        with torch.amp.autocast(device_type="cuda", dtype=torch.float16):
            ys = block(x)
        torch.autograd.backward(ys, gys)
        grads = [p.grad.clone() for p in block.parameters() if p.requires_grad]
        results.append(([y.detach() for y in ys], x.grad.clone(), grads))
        block.zero_grad()
    assert calls == {"fwd": 1, "bwd": 1}
    (ys_g, dx_g, gr_g), (ys_p, dx_p, gr_p) = results
    for a, b in zip(ys_g, ys_p):
        assert a.shape == (2, M // 2, N)
        assert float((a.float() - b.float()).abs().max() / b.float().abs().max()) <= 2e-3
    assert float((dx_g.float() - dx_p.float()).abs().max() / dx_p.float().abs().max()) <= 3e-3
    assert len(gr_g) == 4
    for a, b in zip(gr_g, gr_p):
        assert float((a.float() - b.float()).abs().max() / b.float().abs().max()) <= 3e-3
    # no grad, eval: the same grouped launch for a prefill-sized input; 8 rows go to the grouped GEMV
    grouped.eval(); plain.eval()
    with torch.no_grad():
        for rows in (M, 8):
            x = _t(xh)[:rows]
            for a, b in zip(grouped(x), plain(x)):
                assert float((a.float() - b.float()).abs().max() / b.float().abs().max()) <= 2e-3
    assert calls["fwd"] == 2
    assert ungroup(grouped) == 1 and "_q4_group" not in grouped.k_proj.__dict__
