"""Finetune smoke run (what finetune.py:75-160 of the reference sets up, without peft / Trainer): a loaded
4-bit LLaMA, LoRA adapters on q_proj and v_proj, fp16 autocast, causal-LM loss.
 * the adapter gradients of one step match torch autograd through the dense fp32 model with the same
   adapters written out as plain matmuls;
 * a few AdamW steps reduce the loss and leave every quantized buffer untouched."""
import os

import pytest
import torch

from tiny_llama import GROUPSIZE, build

pytestmark = pytest.mark.gpu


class _DenseLora(torch.nn.Module):
    def __init__(self, lin, A, B, scaling):
        super().__init__()
        self.lin, self.scaling = lin, scaling
        self.A = torch.nn.Parameter(A.clone())
        self.B = torch.nn.Parameter(B.clone())

    def forward(self, x):
        return self.lin(x) + (x @ self.A.t()) @ self.B.t() * self.scaling


def test_lora_finetune_step_matches_dense_autograd_and_trains(tmp_path, oracle):
    from alpaca_lora_4bit_amd import autograd_4bit as ag
    from alpaca_lora_4bit_amd.models import inject_lora_layers
    path = str(tmp_path / "ckpt")
    dense, _ = build(path, oracle, seed=5, with_tokenizer=True)
    model, _ = ag.load_llama_model_4bit_low_ram(path, os.path.join(path, "model.safetensors"), groupsize=GROUPSIZE,
                                                half=True, device_map={"": 0})
    lora = inject_lora_layers(model, target_modules=("q_proj", "v_proj"), r=8, lora_alpha=16)
    assert len(lora) == 4
    torch.manual_seed(0)
    for p in dense.parameters():
        p.requires_grad_(False)
    for name, layer in lora.items():
        B = layer.lora_B["default"].weight
        with torch.no_grad():
            B.copy_(torch.randn_like(B) * 0.05)                  # a trained-looking B: gradients reach A as well
        A = layer.lora_A["default"].weight
        assert A.dtype == torch.float32 and A.requires_grad and B.requires_grad
        parent = dense.get_submodule(name.rsplit(".", 1)[0])
        child = name.rsplit(".", 1)[1]
        setattr(parent, child, _DenseLora(getattr(parent, child), A.detach().cpu(), B.detach().cpu(),
                                          layer.scaling["default"]))
    frozen = {n: b.clone() for n, b in model.named_buffers() if n.endswith(("qweight", "qzeros", "scales", "g_idx"))}
    trainable = [p for p in model.parameters() if p.requires_grad]
    assert len(trainable) == 8 and all(p.dtype == torch.float32 for p in trainable)

    ids = torch.tensor([[1] + [5 + (11 * i) % 200 for i in range(39)], [1] + [9 + (5 * i) % 190 for i in range(39)]])
    loss_scale = 1024.0                                            # fp16 gradients, as under the Trainer's GradScaler

    def loss_of(m, x):
        return m(input_ids=x, labels=x).loss

    with torch.autocast("cuda", dtype=torch.float16):
        loss = loss_of(model, ids.cuda())
    (loss * loss_scale).backward()
    # reference 1: the dense model in fp32 on the CPU (loose: an fp16 model against an fp32 one)
    ref_loss = loss_of(dense, ids)
    ref_loss.backward()
    ref32 = {n: (dense.get_submodule(n).A.grad.clone(), dense.get_submodule(n).B.grad.clone()) for n in lora}
    # reference 2: the same dense model with fp16 weights under the same autocast on the GPU; everything but
    # the quantized matmuls and the adapter kernels is then the same arithmetic (tight)
    dense.zero_grad(set_to_none=True)
    dense16 = dense.cuda()
    for n, mod in dense16.named_modules():
        if not isinstance(mod, _DenseLora) and not list(mod.children()):
            mod.half()
    with torch.autocast("cuda", dtype=torch.float16):
        loss16 = loss_of(dense16, ids.cuda())
    (loss16 * loss_scale).backward()
    assert abs(loss.item() - loss16.item()) <= 5e-3 * abs(loss16.item())
    assert abs(loss.item() - ref_loss.item()) <= 5e-2 * abs(ref_loss.item())
    for name, layer in lora.items():
        d = dense16.get_submodule(name)
        pairs = ((layer.lora_A["default"].weight.grad, d.A.grad, ref32[name][0]),
                 (layer.lora_B["default"].weight.grad, d.B.grad, ref32[name][1]))
        for got, r16, r32 in pairs:
            g = got.float().cpu() / loss_scale
            r16 = r16.float().cpu() / loss_scale
            assert torch.isfinite(g).all() and r32.abs().max() > 0
            e16 = ((g - r16).norm() / r16.norm()).item()
            e32 = ((g - r32).norm() / r32.norm()).item()
            noise = ((r16 - r32).norm() / r32.norm()).item()          # what fp16 alone does to this gradient
            assert e16 <= max(3e-2, 1.5 * noise) and e32 <= max(5e-2, 2.0 * noise), (name, e16, e32, noise)
            print(f"{name}: rel err vs fp16 dense {e16:.4f}, vs fp32 dense {e32:.4f}, fp16-vs-fp32 dense {noise:.4f}")

    opt = torch.optim.AdamW(trainable, lr=2e-3)
    losses = []
    for _ in range(8):
        opt.zero_grad(set_to_none=True)
        with torch.autocast("cuda", dtype=torch.float16):
            loss = loss_of(model, ids.cuda())
        (loss * loss_scale).backward()
        for p in trainable:
            p.grad.div_(loss_scale)
        opt.step()
        losses.append(loss.item())
    assert losses[-1] < losses[0] - 0.05, losses
    for n, b in model.named_buffers():
        if n in frozen:
            assert torch.equal(b, frozen[n]), n
