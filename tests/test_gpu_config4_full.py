"""The full-size LoRA training step of the benchmark definition's configs[4]: random-init 32-layer LLaMA-7B decoder, every
q/k/v/o/gate/up/down projection a 4-bit GPTQ layer (groupsize 128), LoRA r=8 alpha=16 on q_proj and v_proj, one
forward + backward on batch 4 x seq 256 under fp16 autocast, gradient checkpointing off (the reference's flow:
finetune.py:75-104).  Checked: the loss, every adapter gradient, the packed buffers, and -- on inputs captured
inside the running model -- the first and the last 4-bit product against the CPU oracle (1e-2 * max|ref|).
Also the 1024-row products of the MLP up projection (4096 -> 11008) forward and grad-input, whose launch plan
(whole rounds of tiles + a split remainder) only exists at this size."""
import math
import os
import sys

import numpy as np
import pytest
import torch

from conftest import rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _layer_numpy(mod):
    return dict(qweight=mod.qweight.cpu().numpy(), qzeros=mod.qzeros.cpu().numpy(),
                scales=mod.scales.cpu().numpy(), g_idx=mod.g_idx.cpu().numpy())


def test_llama7b_lora_step_full_size(oracle):
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import bench
    from alpaca_lora_4bit_amd import autograd_4bit as ag
    from alpaca_lora_4bit_amd.models import Linear4bitLt, inject_lora_layers
    gen = torch.Generator(device="cuda").manual_seed(11)
    model = bench._random_llama7b(gen, 32)
    lora = inject_lora_layers(model, target_modules=("q_proj", "v_proj"), r=8, lora_alpha=16)
    assert len(lora) == 64
    with torch.no_grad():
        for l in lora.values():
            l.lora_B["default"].weight.normal_(0, 0.02, generator=gen)
    quant = [m for m in model.modules() if isinstance(m, ag.Autograd4bitQuantLinear)]
    assert len(quant) == 224
    sums = [(int(m.qweight.sum(dtype=torch.int64)), int(m.qzeros.sum(dtype=torch.int64)),
             float(m.scales.float().sum())) for m in quant]
    ids = torch.randint(0, 32000, (4, 256), device="cuda", generator=gen)
    model.train()
    model.config.use_cache = False

    first = model.model.layers[0].self_attn.q_proj
    last = model.model.layers[31].mlp.down_proj
    assert isinstance(first, Linear4bitLt) and not isinstance(last, Linear4bitLt)
    seen = {}
    hooks = [first.register_forward_hook(lambda m, i, o: seen.__setitem__("first", (i[0].detach(), o.detach()))),
             last.register_forward_hook(lambda m, i, o: seen.__setitem__("last", (i[0].detach(), o.detach())))]
    with torch.amp.autocast(device_type="cuda", dtype=torch.float16):
        loss = model(input_ids=ids, labels=ids).loss
    # fp16 gradients need the loss scaled: 65536 is where the fp16 Trainer's GradScaler starts.  (At 1024 the rank-8
    # projection dy @ B of one q_proj, whose gradients are tiny in an untrained model, underflows fp16 to zero --
    # in the reference's composition just as here.)
    (loss * 65536.0).backward()
    torch.cuda.synchronize()
    for h in hooks:
        h.remove()

    # untrained model, uniform random tokens: the loss sits near ln(vocabulary)
    assert math.isfinite(loss.item()) and abs(loss.item() - math.log(32000)) < 1.5, loss.item()
    grads = [p.grad for l in lora.values() for p in (l.lora_A["default"].weight, l.lora_B["default"].weight)]
    assert len(grads) == 128
    for g in grads:
        assert g is not None and bool(torch.isfinite(g).all()) and float(g.abs().max()) > 0
    for m, s in zip(quant, sums):
        assert (int(m.qweight.sum(dtype=torch.int64)), int(m.qzeros.sum(dtype=torch.int64)),
                float(m.scales.float().sum())) == s

    # the products inside the model against the oracle, on a sample of the 1024 token rows (oracle time)
    rows = np.arange(0, 1024, 8)
    xin, yout = seen["first"]
    assert xin.shape == (4, 256, 4096) and yout.shape == (4, 256, 4096)
    x = xin.reshape(-1, 4096).half().cpu().numpy()[rows]
    lay = _layer_numpy(first)
    W = oracle.dequant_v2(lay["qweight"], lay["qzeros"], lay["scales"], lay["g_idx"])
    A = first.lora_A["default"].weight.detach().float().cpu().numpy()
    B = first.lora_B["default"].weight.detach().float().cpu().numpy()
    ref = oracle.lora_forward(x, W, A, B, first.scaling["default"])
    assert rel_err(yout.reshape(-1, 4096).float().cpu().numpy()[rows], ref) <= TOL
    xin, yout = seen["last"]
    assert xin.shape == (4, 256, 11008) and yout.shape == (4, 256, 4096)
    x = xin.reshape(-1, 11008).half().cpu().numpy()[rows]
    lay = _layer_numpy(last)
    ref = oracle.matmul_recons(x, lay["qweight"], lay["qzeros"], lay["scales"], lay["g_idx"])
    assert np.abs(ref).max() > 0
    assert rel_err(yout.reshape(-1, 4096).float().cpu().numpy()[rows], ref) <= TOL
    del model, lora, quant, grads
    torch.cuda.empty_cache()


def test_mlp_up_projection_1024_rows_fwd_and_grad_input(oracle):
    from alpaca_lora_4bit_amd import quant_hip
    K, N, M = 4096, 11008, 1024
    layer = oracle.make_layer(K, N, 128, seed=41)
    t = {k: torch.from_numpy(layer[k]).cuda() for k in ("qweight", "qzeros", "scales", "g_idx")}
    x = oracle.make_activations(M, K, seed=42)
    dy = oracle.make_activations(M, N, seed=43)
    y = quant_hip.gemm_fwd(torch.from_numpy(x).cuda(), t["qweight"], t["qzeros"], t["scales"], None, 128)
    dx = quant_hip.gemm_bwd_dx(torch.from_numpy(dy).cuda(), t["qweight"], t["qzeros"], t["scales"], None, 128)
    torch.cuda.synchronize()
    # every element against the library's own bit-exact dense W (checked against the oracle elsewhere) ...
    W = quant_hip.dequant(t["qweight"], t["qzeros"], t["scales"], None, 128).float()
    ref_y = torch.from_numpy(x).cuda().float() @ W
    ref_dx = torch.from_numpy(dy).cuda().float() @ W.t()
    assert float((y.float() - ref_y).abs().max() / ref_y.abs().max()) <= TOL
    assert float((dx.float() - ref_dx).abs().max() / ref_dx.abs().max()) <= TOL
    # ... and a sample of rows (spread over all four 256-row tiles) against the CPU oracle itself
    rows = np.arange(3, M, 16)
    ref = oracle.matmul_recons(x[rows], layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    assert rel_err(y.cpu().numpy()[rows], ref) <= TOL
    ref = oracle.matmul_recons_t(dy[rows], layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    assert rel_err(dx.cpu().numpy()[rows], ref) <= TOL
