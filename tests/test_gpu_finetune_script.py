"""The finetune and inference flows end to end on the GPU (the reference's finetune.py / inference.py as modules):
command line -> packed-model loader -> LoRA injection -> dataset reader -> transformers.Trainer under fp16 autocast
-> adapter files -> generation with the adapter applied.  Model: the synthetic 2-block LLaMA of tiny_llama.py."""
import json
import os
import random

import pytest
import torch

from tiny_llama import GROUPSIZE, build

pytestmark = pytest.mark.gpu

WORDS = ["alpha", "beta", "gamma", "delta", "lora", "quant", "weight", "matrix", "token", "layer", "the", "of"]


def _corpus(path, lines=48):
    rnd = random.Random(1)
    with open(path, "w") as fh:
        for _ in range(lines):
            # a strongly repetitive pattern: a few steps of LoRA training must lower its loss
            start = rnd.randrange(len(WORDS))
            fh.write(" ".join(WORDS[(start + j) % len(WORDS)] for j in range(10)) + "\n")


@pytest.mark.parametrize("grad_chckpt", [False, True])
def test_finetune_module_trains_and_saves_an_adapter(tmp_path, oracle, grad_chckpt):
    from safetensors.torch import load_file
    from alpaca_lora_4bit_amd import finetune
    ckpt = str(tmp_path / "ckpt")
    build(ckpt, oracle, seed=5, with_tokenizer=True)
    data = str(tmp_path / "data.txt")
    _corpus(data)
    out = str(tmp_path / "lora_out")
    argv = [data, "--ds_type", "txt", "--llama_q4_config_dir", ckpt, "--llama_q4_model",
            os.path.join(ckpt, "model.safetensors"), "--groupsize", str(GROUPSIZE), "--lora_out_dir", out,
            "--mbatch_size", "4", "--batch_size", "8", "--epochs", "3", "--lr", "5e-3", "--cutoff_len", "24",
            "--warmup_steps", "1", "--logging_steps", "1", "--val_set_size", "0", "--lora_dropout", "0.0"]
    if grad_chckpt:
        argv += ["--grad_chckpt", "--grad_chckpt_ratio", "0.5"]
    model, tokenizer, trainer = finetune.main(argv)

    losses = [h["loss"] for h in trainer.state.log_history if "loss" in h]
    assert len(losses) >= 6 and all(l == l for l in losses)                 # 48 rows / 8 per step * 3 epochs; no NaN
    # only rank-8 adapters on q_proj / v_proj of a random model train: the loss falls slowly but steadily
    assert sum(losses[-3:]) / 3 < sum(losses[:3]) / 3 - 0.1, losses
    lora = [m for m in model.modules() if "Linear4bitLt" in str(type(m))]
    assert len(lora) == 4                                                   # q_proj, v_proj of two blocks
    assert all(float(m.lora_B["default"].weight.detach().abs().max()) > 0 for m in lora)      # B starts at zero
    assert all(m.qweight.dtype == torch.int32 and m.scales.dtype == torch.float16 for m in lora)
    if grad_chckpt:
        assert [hasattr(l, "old_forward_for_cp") for l in model.model.layers] == [True, False]   # int(2 * 0.5) = 1 block

    saved = load_file(os.path.join(out, "adapter_model.safetensors"))
    assert len(saved) == 8 and all(k.startswith("base_model.model.model.layers.") for k in saved)
    name = "model.layers.1.self_attn.v_proj"
    live = dict(model.named_modules())[name]
    assert torch.equal(saved[f"base_model.model.{name}.lora_B.weight"], live.lora_B["default"].weight.detach().cpu())
    cfg = json.load(open(os.path.join(out, "adapter_config.json")))
    assert cfg["r"] == 8 and cfg["lora_alpha"] == 16 and cfg["target_modules"] == ["q_proj", "v_proj"]

    if not grad_chckpt:
        # generation through the inference flow, with and without the adapter
        from alpaca_lora_4bit_amd import inference
        base_args = [ckpt, os.path.join(ckpt, "model.safetensors"), "--groupsize", str(GROUPSIZE), "--prompt",
                     "alpha beta gamma", "--max_new_tokens", "6", "--greedy"]
        text_lora, _ = inference.main(base_args + ["--lora", out])
        text_base, _ = inference.main(base_args)
        assert isinstance(text_lora, str) and text_lora.startswith("alpha beta gamma")
        assert text_base.startswith("alpha beta gamma")


def test_finetune_module_on_alpaca_records_with_evaluation(tmp_path, oracle):
    """Alpaca-style JSON records, a validation split and periodic evaluation (no-grad forward of the LoRA layers with
    many rows) through the same flow."""
    from alpaca_lora_4bit_amd import finetune
    ckpt = str(tmp_path / "ckpt")
    build(ckpt, oracle, seed=6, with_tokenizer=True)
    rnd = random.Random(2)
    records = [{"instruction": " ".join(rnd.choice(WORDS) for _ in range(4)), "input": "",
                "output": " ".join(rnd.choice(WORDS) for _ in range(6))} for _ in range(40)]
    data = str(tmp_path / "alpaca.json")
    with open(data, "w") as fh:
        json.dump(records, fh)
    out = str(tmp_path / "lora_out")
    model, tokenizer, trainer = finetune.main([
        data, "--ds_type", "alpaca", "--llama_q4_config_dir", ckpt, "--llama_q4_model",
        os.path.join(ckpt, "model.safetensors"), "--groupsize", str(GROUPSIZE), "--lora_out_dir", out,
        "--mbatch_size", "4", "--batch_size", "4", "--epochs", "1", "--lr", "1e-3", "--cutoff_len", "96",
        "--warmup_steps", "1", "--logging_steps", "2", "--val_set_size", "0.2", "--lora_dropout", "0.05"])
    evals = [h["eval_loss"] for h in trainer.state.log_history if "eval_loss" in h]
    losses = [h["loss"] for h in trainer.state.log_history if "loss" in h]
    assert evals and all(e == e and e > 0 for e in evals) and losses and all(l == l for l in losses)
    assert os.path.exists(os.path.join(out, "adapter_model.safetensors"))


@pytest.mark.parametrize("act_order", [False, True])
def test_hip_graph_decode_gives_the_eager_tokens(tmp_path, oracle, act_order):
    """inference.greedy_generate_graph: every replay of the captured one-token step (with host reads and eager
    copies between the replays) must pick the token that transformers' eager `generate` picks; plain layers, fused
    q+k+v / gate+up layers, and the command-line flow with an adapter."""
    from alpaca_lora_4bit_amd import autograd_4bit as ag, inference
    from alpaca_lora_4bit_amd.model_attn_mlp_patch import make_fused_mlp, make_quant_attn
    ckpt = str(tmp_path / "ckpt")
    build(ckpt, oracle, act_order=act_order, seed=8, with_tokenizer=True)
    weights = os.path.join(ckpt, "model.safetensors")
    model, tokenizer = ag.load_llama_model_4bit_low_ram(ckpt, weights, groupsize=GROUPSIZE, half=True, device_map={"": 0})
    ids = torch.tensor([[1] + [7 + (13 * i) % 180 for i in range(9)]]).cuda()
    new = 24
    for fused in (False, True):
        if fused:
            # grouped in place; act-order projections carry their own row permutations, so their groups find at the
            # first call that they cannot share one launch and every member keeps its own
            assert make_quant_attn(model) == 2 and make_fused_mlp(model) == 2
        with torch.no_grad():
            want = model.generate(input_ids=ids, max_new_tokens=new, min_new_tokens=new, do_sample=False)
        # eos id -1 never matches: it makes the loop read every token on the host between two replays
        got = inference.greedy_generate_graph(model, ids, new, eos_token_id=-1 if fused else None)
        assert got.shape == want.shape == (1, ids.shape[1] + new)
        assert got.tolist() == want.tolist()
        assert len(set(want[0, ids.shape[1]:].tolist())) > 3             # not a degenerate constant continuation
    # layers with a LoRA adapter (the three-launch decode path of Linear4bitLt) inside the captured step
    from alpaca_lora_4bit_amd import models
    lora_model, _ = ag.load_llama_model_4bit_low_ram(ckpt, weights, groupsize=GROUPSIZE, half=True, device_map={"": 0})
    layers = models.inject_lora_layers(lora_model, target_modules=("q_proj", "v_proj"), r=8, lora_alpha=16)
    gen = torch.Generator(device="cuda").manual_seed(3)
    with torch.no_grad():
        for l in layers.values():
            l.lora_B["default"].weight.normal_(0, 0.2, generator=gen)
    lora_model.eval()
    with torch.no_grad(), torch.amp.autocast(device_type="cuda"):
        want = lora_model.generate(input_ids=ids, max_new_tokens=new, min_new_tokens=new, do_sample=False)
        got = inference.greedy_generate_graph(lora_model, ids, new)
    assert got.tolist() == want.tolist()
    # the flow from the command line with --fuse and --hip_graph: plain argmax decoding (no repetition penalty)
    args = [ckpt, weights, "--groupsize", str(GROUPSIZE), "--prompt", "alpha beta gamma", "--max_new_tokens", "12",
            "--greedy"]
    prompt = tokenizer("alpha beta gamma", return_tensors="pt", add_special_tokens=False)["input_ids"].cuda()
    with torch.no_grad():
        want = model.generate(input_ids=prompt, max_new_tokens=12, do_sample=False,
                              eos_token_id=getattr(tokenizer, "eos_token_id", None))
    text_graph, _ = inference.main(args + ["--fuse", "--hip_graph"])
    assert text_graph == tokenizer.decode(want[0].tolist())
    # sampling (the reference's settings) between the replays: same draws as the same loop without capture
    sampling = {k: inference.SAMPLING[k] for k in ("repetition_penalty", "temperature", "top_k", "top_p")}
    runs = []
    for use_graph in (True, False, True):
        torch.manual_seed(1234)
        runs.append(inference.generate_graph(model, ids, new, sampling=sampling, use_graph=use_graph).tolist())
    assert runs[0] == runs[1] == runs[2]
    assert runs[0] != inference.greedy_generate_graph(model, ids, new).tolist()
    text_sampled, _ = inference.main(args[:-1] + ["--hip_graph"])
    assert text_sampled.startswith("alpha beta gamma")
