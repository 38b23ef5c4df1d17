"""Synthetic LLaMA checkpoint for the loader tests: a tiny config, GPTQ-packed Linear layers written
as `<module>.qweight / qzeros / scales / g_idx` into a safetensors file (the on-disk format the
reference's loaders read, autograd_4bit.py:250-287), a sentencepiece tokenizer trained on the spot,
and the matching dense fp32 model (weights = the oracle's dequantized W) to compare against."""
import json
import os
import random

import numpy as np
import torch

HIDDEN, INTER, LAYERS, HEADS, GROUPSIZE = 256, 512, 2, 4, 128


def _train_tokenizer(path):
    import sentencepiece as spm
    rnd = random.Random(0)
    words = ["alpha", "beta", "gamma", "delta", "lora", "quant", "weight", "matrix", "token", "layer", "the", "of",
             "and", "model", "group", "scale", "zero", "bit", "four", "gpu", "wave", "front", "kernel", "fast"]
    corpus = os.path.join(path, "corpus.txt")
    with open(corpus, "w") as f:
        for _ in range(1500):
            f.write(" ".join(rnd.choice(words) for _ in range(rnd.randint(3, 12))) + "\n")
    spm.SentencePieceTrainer.train(input=corpus, model_prefix=os.path.join(path, "tokenizer"), vocab_size=320,
                                   model_type="bpe", hard_vocab_limit=False, bos_id=1, eos_id=2, unk_id=0, pad_id=-1,
                                   minloglevel=2)
    os.remove(corpus)


def build(path, oracle, act_order=False, seed=0, with_tokenizer=True):
    """Writes config.json, model.safetensors (+ tokenizer.model) into `path`.
    Returns (dense_model_fp32, {module_name: oracle layer dict})."""
    from safetensors.torch import save_file
    from transformers import LlamaConfig, LlamaForCausalLM
    os.makedirs(path, exist_ok=True)
    if with_tokenizer:
        _train_tokenizer(path)
    config = LlamaConfig(vocab_size=320, hidden_size=HIDDEN, intermediate_size=INTER, num_hidden_layers=LAYERS,
                         num_attention_heads=HEADS, num_key_value_heads=HEADS, max_position_embeddings=128,
                         tie_word_embeddings=False, bos_token_id=1, eos_token_id=2)
    config.save_pretrained(path)
    torch.manual_seed(seed)
    dense = LlamaForCausalLM(config).float().eval()
    state = {k: v.clone() for k, v in dense.state_dict().items()}
    layers = {}
    i = 0
    for name, mod in dense.named_modules():
        if isinstance(mod, torch.nn.Linear) and name != "lm_head":
            K, N = mod.in_features, mod.out_features
            L = oracle.make_layer(K, N, GROUPSIZE, act_order=act_order, seed=seed * 100 + i)
            i += 1
            # scales sized so that a layer has about unit gain (W entries ~ 6.5 * scale): the model then stays in
            # a regime where fp16 and fp32 runs agree closely and comparisons are meaningful
            L["scales"] = (L["scales"].astype(np.float32) * (0.15 / np.sqrt(K) / 0.0125)).astype(np.float16)
            W = oracle.dequant_v2(L["qweight"], L["qzeros"], L["scales"], L["g_idx"]).astype(np.float32)
            with torch.no_grad():
                mod.weight.copy_(torch.from_numpy(W.T.copy()))
            del state[name + ".weight"]
            state[name + ".qweight"] = torch.from_numpy(L["qweight"].astype(np.int32))
            state[name + ".qzeros"] = torch.from_numpy(L["qzeros"].astype(np.int32))
            state[name + ".scales"] = torch.from_numpy(L["scales"])
            state[name + ".g_idx"] = torch.from_numpy(L["g_idx"].astype(np.int32))
            layers[name] = L
    save_file({k: v.contiguous() for k, v in state.items()}, os.path.join(path, "model.safetensors"))
    return dense, layers
