"""Loaders (autograd_4bit.py:250-360 of the reference): structure and buffers on the CPU; logits of the
loaded model on the GPU against a dense fp32 model holding the oracle's dequantized weights."""
import os

import numpy as np
import pytest
import torch

from tiny_llama import GROUPSIZE, build


@pytest.fixture(scope="module")
def checkpoint(tmp_path_factory, oracle):
    path = str(tmp_path_factory.mktemp("tiny_llama"))
    dense, layers = build(path, oracle)
    return path, dense, layers


def test_loader_builds_quantized_skeleton_and_fills_buffers(checkpoint):
    from alpaca_lora_4bit_amd import autograd_4bit as ag
    path, dense, layers = checkpoint
    model, tokenizer = ag.load_llama_model_4bit_low_ram(path, os.path.join(path, "model.safetensors"),
                                                        groupsize=GROUPSIZE, device_map={"": "cpu"}, seqlen=77)
    assert model.seqlen == 77 and tokenizer.truncation_side == "left"
    assert isinstance(model.lm_head, torch.nn.Linear)                 # lm_head stays dense (autograd_4bit.py:261-263)
    quant = {n: m for n, m in model.named_modules() if isinstance(m, ag.Autograd4bitQuantLinear)}
    assert set(quant) == set(layers) and len(quant) == 7 * 2
    for n, m in quant.items():
        L = layers[n]
        assert m.groupsize == GROUPSIZE and m.bits == 4 and not m.is_v1_model
        assert m.qweight.dtype == torch.int32 and torch.equal(m.qweight, torch.from_numpy(L["qweight"].astype(np.int32)))
        assert torch.equal(m.qzeros, torch.from_numpy(L["qzeros"].astype(np.int32)))
        assert torch.equal(m.g_idx, torch.from_numpy(L["g_idx"].astype(np.int32)))
        assert torch.equal(m.scales.half(), torch.from_numpy(L["scales"]))        # fp16 values survive the fp32 buffer
        assert float(m.bias.abs().max()) == 0.0                                   # absent from the file: stays zero
    assert not any(p.is_meta for p in model.parameters())
    assert torch.equal(model.model.embed_tokens.weight, dense.model.embed_tokens.weight)


def test_loader_half_casts_buffers(checkpoint):
    from alpaca_lora_4bit_amd import autograd_4bit as ag
    path, _, _ = checkpoint
    model, _ = ag.load_llama_model_4bit_low_ram(path, os.path.join(path, "model.safetensors"), groupsize=GROUPSIZE,
                                                half=True, device_map={"": "cpu"})
    for m in model.modules():
        if isinstance(m, ag.Autograd4bitQuantLinear):
            assert m.scales.dtype == torch.float16 and m.bias.dtype == torch.float16 and m.qweight.dtype == torch.int32
    assert model.lm_head.weight.dtype == torch.float16


def test_offload_alias_and_missing_peft_message(checkpoint):
    from alpaca_lora_4bit_amd import autograd_4bit as ag
    assert ag.load_llama_model_4bit_low_ram_and_offload_to_cpu is ag.load_llama_model_4bit_low_ram_and_offload
    with pytest.raises(AttributeError):
        ag.no_such_loader


@pytest.mark.gpu
@pytest.mark.parametrize("act_order", [False, True])
def test_loaded_model_logits_match_dense_reference(tmp_path, oracle, act_order):
    """Prefill of 24 tokens (fused GEMM path) and a 1-token step (GEMV path) through the loaded model."""
    from alpaca_lora_4bit_amd import autograd_4bit as ag
    path = str(tmp_path / "ckpt")
    dense, _ = build(path, oracle, act_order=act_order, seed=3, with_tokenizer=True)
    model, tokenizer = ag.load_llama_model_4bit_low_ram(path, os.path.join(path, "model.safetensors"),
                                                        groupsize=GROUPSIZE, half=True, device_map={"": 0})
    ids = torch.tensor([[1] + [5 + (7 * i) % 200 for i in range(23)]])
    with torch.no_grad():
        ref = dense(ids).logits.float()
        ref1 = dense(ids[:, :1]).logits.float()
        got = model(ids.cuda()).logits.float().cpu()
        got1 = model(ids[:, :1].cuda()).logits.float().cpu()
        # the same dense model in fp16 on the GPU: everything but the quantized matmuls is then identical
        # arithmetic (attention, norms, lm_head), so this comparison isolates the 4-bit layers
        dense16 = dense.half().cuda()
        h = dense16(ids.cuda()).logits.float().cpu()
        h1 = dense16(ids[:, :1].cuda()).logits.float().cpu()
    for g, r16, r32 in ((got, h, ref), (got1, h1, ref1)):
        assert g.shape == r32.shape
        scale = r32.abs().max().item()
        assert (g - r16).abs().max().item() <= 1e-2 * scale
        assert (g - r32).abs().max().item() <= 1e-1 * scale        # fp16 model against the fp32 one
    # generation runs end to end (greedy, a few tokens) and agrees with the dense model's first choice
    out = model.generate(ids.cuda(), max_new_tokens=3, do_sample=False)
    assert out.shape == (1, 27)
    assert int(out[0, 24]) == int(ref[0, -1].argmax())


@pytest.mark.gpu
def test_fused_qkv_and_gate_up_keep_the_logits(tmp_path, oracle):
    """make_quant_attn / make_fused_mlp with the reference's N-concatenated layout (model_attn_mlp_patch.py:73-247):
    three / two projections become one launch each; the model's own attention and MLP code keeps running on slice views."""
    from alpaca_lora_4bit_amd import autograd_4bit as ag
    from alpaca_lora_4bit_amd.model_attn_mlp_patch import FusedProjectionSlice, make_fused_mlp, make_quant_attn
    path = str(tmp_path / "ckpt")
    build(path, oracle, seed=4, with_tokenizer=True)
    model, _ = ag.load_llama_model_4bit_low_ram(path, os.path.join(path, "model.safetensors"), groupsize=GROUPSIZE,
                                                half=True, device_map={"": 0})
    ids = torch.tensor([[1] + [5 + (7 * i) % 200 for i in range(23)]]).cuda()
    with torch.no_grad():
        before, before1 = model(ids).logits.float(), model(ids[:, :1]).logits.float()
    n_quant = sum(isinstance(m, ag.Autograd4bitQuantLinear) for m in model.modules())
    assert make_quant_attn(model, concatenate=True) == 2 and make_fused_mlp(model, concatenate=True) == 2
    layer0 = model.model.layers[0]
    assert isinstance(layer0.self_attn.q_proj, FusedProjectionSlice) and isinstance(layer0.mlp.up_proj, FusedProjectionSlice)
    assert layer0.self_attn.qkv_proj.out_features == 3 * 256 and layer0.mlp.gate_up_proj.out_features == 2 * 512
    assert sum(isinstance(m, ag.Autograd4bitQuantLinear) for m in model.modules()) == n_quant - 2 * 3   # 5 -> 2 per block
    assert not any(k.endswith("q_proj.qweight") for k in model.state_dict())                          # no duplicate state
    with torch.no_grad():
        after, after1 = model(ids).logits.float(), model(ids[:, :1]).logits.float()
    for a, b in ((after, before), (after1, before1)):
        assert (a - b).abs().max().item() <= 2e-3 * b.abs().max().item()
    assert make_quant_attn(model, concatenate=True) == 0     # idempotent: nothing left to fuse
    # the slices in any order, one fused launch per input; an in-place change of the input is noticed; nothing stays
    # cached once the block has returned
    attn = layer0.self_attn
    calls = []
    handle = attn.qkv_proj.register_forward_hook(lambda m, i, o: calls.append(1))
    x = torch.randn(1, 3, 256, device="cuda", dtype=torch.float16)
    with torch.no_grad():
        v, q, k = attn.v_proj(x), attn.q_proj(x), attn.k_proj(x)
        assert len(calls) == 1
        full = attn.qkv_proj(x)
        assert torch.equal(torch.cat([q, k, v], dim=-1), full)
        x.mul_(2.0)
        q2 = attn.q_proj(x)
        assert len(calls) == 3 and not torch.equal(q2, q)
        model(ids[:, :1])
    handle.remove()
    assert attn.q_proj._group._x is None and attn.q_proj._group._y is None


@pytest.mark.gpu
def test_projections_grouped_in_place_keep_the_logits_with_and_without_adapters(tmp_path, oracle, monkeypatch):
    """make_quant_attn / make_fused_mlp in their default, in-place form: q|k|v and gate|up stay on their own tensors and
    at decode sizes share ONE grouped launch (q4_gemv_grouped_f16); the MLP decode step is one launch
    (q4_mlp_decode_f16); LoRA layers on q_proj / v_proj stay members of their group.  Logits against the unfused model
    (and through it the dense model of test_load_and_run...), at prefill and at one decode row."""
    import json
    from safetensors.torch import save_file
    from alpaca_lora_4bit_amd import autograd_4bit as ag, finetune, models, quant_hip
    from alpaca_lora_4bit_amd.model_attn_mlp_patch import inject_lora_layers as inject_saved
    from alpaca_lora_4bit_amd.model_attn_mlp_patch import make_fused_mlp, make_quant_attn, ungroup
    path = str(tmp_path / "ckpt")
    build(path, oracle, seed=5, with_tokenizer=True)
    load = lambda: ag.load_llama_model_4bit_low_ram(path, os.path.join(path, "model.safetensors"), groupsize=GROUPSIZE,
                                                    half=True, device_map={"": 0})[0]
    ids = torch.tensor([[1] + [5 + (7 * i) % 200 for i in range(23)]]).cuda()
    model = load()
    keys = sorted(model.state_dict())
    with torch.no_grad():
        before, before1 = model(ids).logits.float(), model(ids[:, :1]).logits.float()
    assert make_quant_attn(model) == 2 and make_fused_mlp(model) == 2
    assert make_quant_attn(model) == 0 and make_fused_mlp(model) == 0          # idempotent
    assert sorted(model.state_dict()) == keys                                 # same modules, same tensors, same keys
    calls = {"grouped": 0, "mlp": 0, "gemv": 0}
    for name, key in (("gemv_grouped_prepared", "grouped"), ("mlp_decode_prepared", "mlp"), ("gemv", "gemv")):
        real = getattr(quant_hip, name)
        monkeypatch.setattr(quant_hip, name, (lambda real, key: lambda *a, **k: (calls.__setitem__(key, calls[key] + 1), real(*a, **k))[1])(real, key))
    with torch.no_grad():
        after, after1 = model(ids).logits.float(), model(ids[:, :1]).logits.float()
    # one decode row through 2 blocks: q|k|v grouped once per block, the MLP in one launch, o_proj alone
    assert calls == {"grouped": 2, "mlp": 2, "gemv": 2}
    for a, b in ((after, before), (after1, before1)):
        assert (a - b).abs().max().item() <= 3e-3 * b.abs().max().item()
    assert not quant_hip.mlp_decode_gave_up()
    # the members in any order and more than once; an in-place change of the input is noticed
    attn = model.model.layers[0].self_attn
    x = torch.randn(1, 2, 256, device="cuda", dtype=torch.float16)
    plain = load().model.layers[0].self_attn
    with torch.no_grad():
        for name in ("v_proj", "q_proj", "k_proj", "q_proj"):
            assert torch.equal(getattr(attn, name)(x), getattr(plain, name)(x))
        x.mul_(2.0)
        assert torch.equal(attn.k_proj(x), plain.k_proj(x))
        model(ids[:, :1])
    assert attn.q_proj.__dict__["_q4_group"]._x is None

    # a saved q/v adapter on the grouped model against the same adapter on an ungrouped one
    r, alpha = 8, 16
    gen = torch.Generator().manual_seed(12)
    folder = str(tmp_path / "lora")
    os.makedirs(folder)
    state = {}
    for i in range(2):
        for proj in ("q_proj", "v_proj"):
            base = f"base_model.model.model.layers.{i}.self_attn.{proj}"
            state[f"{base}.lora_A.weight"] = (torch.randn(r, 256, generator=gen) * 0.05).float()
            state[f"{base}.lora_B.weight"] = (torch.randn(256, r, generator=gen) * 0.06).float()
    save_file(state, os.path.join(folder, "adapter_model.safetensors"))
    json.dump({"r": r, "lora_alpha": alpha, "peft_type": "LORA"}, open(os.path.join(folder, "adapter_config.json"), "w"))
    layers = inject_saved(model, folder)
    assert len(layers) == 4 and all(isinstance(l, models.Linear4bitLt) for l in layers)
    assert attn.q_proj.__dict__["_q4_group"] is attn.k_proj.__dict__["_q4_group"] is attn.v_proj.__dict__["_q4_group"]
    ref = load()
    models.inject_lora_layers(ref, target_modules=("q_proj", "v_proj"), r=r, lora_alpha=alpha)
    assert finetune.load_adapter(ref, folder) == 8
    ref.half()
    calls.update(grouped=0, mlp=0, gemv=0)
    with torch.no_grad():
        for rows in (ids, ids[:, :1]):
            want, got = ref(rows).logits.float(), model(rows).logits.float()
            assert (got - want).abs().max().item() <= 4e-3 * want.abs().max().item()
        assert (ref(ids).logits.float() - before).abs().max().item() > 0.05 * before.abs().max().item()   # the adapter matters
    assert calls["grouped"] == 2 and calls["mlp"] == 2                        # the LoRA members still share the launch
    assert ungroup(model) == 4 and "_q4_group" not in attn.q_proj.__dict__
    with torch.no_grad():
        again = model(ids[:, :1]).logits.float()
    assert (again - ref(ids[:, :1]).logits.float()).abs().max().item() <= 4e-3 * again.abs().max().item()


@pytest.mark.gpu
def test_saved_adapter_injected_on_fused_qkv(tmp_path, oracle):
    """inject_lora_layers(model, lora_path) (model_attn_mlp_patch.py:283-335 of the reference): a saved q/v adapter
    lands on the fused qkv layer as one block-structured adapter; logits equal those of the unfused model carrying
    the same adapter on q_proj and v_proj, at prefill and at one decode row, and a second call replaces the first."""
    import json
    from safetensors.torch import save_file
    from alpaca_lora_4bit_amd import autograd_4bit as ag, finetune, models
    from alpaca_lora_4bit_amd.model_attn_mlp_patch import inject_lora_layers as inject_saved, make_quant_attn
    path = str(tmp_path / "ckpt")
    build(path, oracle, seed=6, with_tokenizer=True)
    load = lambda: ag.load_llama_model_4bit_low_ram(path, os.path.join(path, "model.safetensors"), groupsize=GROUPSIZE,
                                                    half=True, device_map={"": 0})[0]
    r, alpha = 8, 16
    gen = torch.Generator().manual_seed(11)

    def write_adapter(folder, scale):
        os.makedirs(folder)
        state = {}
        for i in range(2):
            for proj in ("q_proj", "v_proj"):
                base = f"base_model.model.model.layers.{i}.self_attn.{proj}"
                state[f"{base}.lora_A.weight"] = (torch.randn(r, 256, generator=gen) * 0.05).float()
                state[f"{base}.lora_B.weight"] = (torch.randn(256, r, generator=gen) * scale).float()
        save_file(state, os.path.join(folder, "adapter_model.safetensors"))
        json.dump({"r": r, "lora_alpha": alpha, "peft_type": "LORA"}, open(os.path.join(folder, "adapter_config.json"), "w"))

    first, second = str(tmp_path / "lora_a"), str(tmp_path / "lora_b")
    write_adapter(first, 0.05)
    write_adapter(second, 0.08)
    ids = torch.tensor([[1] + [5 + (11 * i) % 200 for i in range(23)]]).cuda()

    fused = load()
    with torch.no_grad():
        plain = fused(ids).logits.float()
    assert make_quant_attn(fused, concatenate=True) == 2
    for folder in (first, second):                                          # the second call replaces the first adapter
        layers = inject_saved(fused, folder)
        assert len(layers) == 2 and all(l.lora_A["default"].weight.shape == (2 * r, 256) for l in layers)
        assert all(abs(l.scaling["default"] - alpha / r) < 1e-12 for l in layers)
        k_rows = layers[0].lora_B["default"].weight[256:512]
        assert float(k_rows.abs().max()) == 0.0                             # nothing lands on k_proj
        ref = load()
        models.inject_lora_layers(ref, target_modules=("q_proj", "v_proj"), r=r, lora_alpha=alpha)
        assert finetune.load_adapter(ref, folder) == 8
        ref.half()
        with torch.no_grad():
            for rows in (ids, ids[:, :1]):
                want, got = ref(rows).logits.float(), fused(rows).logits.float()
                assert (got - want).abs().max().item() <= 4e-3 * want.abs().max().item()
        assert (ref(ids).logits.float() - plain).abs().max().item() > 0.05 * plain.abs().max().item()   # the adapter matters
