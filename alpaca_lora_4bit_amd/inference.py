"""Text generation with a 4-bit GPTQ LLaMA: the flow of the reference's top-level inference.py:1-49 as a module,

    python -m alpaca_lora_4bit_amd.inference ./llama-7b-4bit/ ./llama-7b-4bit/model.safetensors --groupsize 128 \\
        --prompt "I think the meaning of life is"

Steps as in the reference: load the packed model, `model.half()` and halve `scales` / `bias` (v1: `zeros`) of every
4-bit layer (`:15-22`), wrap `generate` in autocast (`:24-27`), sample with the reference's settings (`:33-44`:
temperature 0.9, top-p 0.95, top-k 40, repetition penalty 1.1, 20 new tokens), print the text and the seconds taken.
`--lora` applies an adapter directory written by `alpaca_lora_4bit_amd.finetune` (or by peft) first.
"""
import argparse
import time

import torch

SAMPLING = dict(do_sample=True, use_cache=True, repetition_penalty=1.1, temperature=0.9, top_p=0.95, top_k=40,
                return_dict_in_generate=True, output_attentions=False, output_hidden_states=False,
                output_scores=False)


def _parse(argv):
    p = argparse.ArgumentParser(description="Generate text with a 4-bit GPTQ LLaMA")
    p.add_argument("config_path", nargs="?", default="./llama-13b-4bit/")
    p.add_argument("model_path", nargs="?", default="./llama-13b-4bit.pt")
    p.add_argument("--groupsize", type=int, default=-1)
    p.add_argument("--v1", action="store_true")
    p.add_argument("--lora", default=None, help="adapter directory to apply")
    p.add_argument("--lora_r", type=int, default=8)
    p.add_argument("--lora_alpha", type=int, default=16)
    p.add_argument("--prompt", default="I think the meaning of life is")
    p.add_argument("--max_new_tokens", type=int, default=20)
    p.add_argument("--greedy", action="store_true", help="argmax decoding instead of sampling")
    return p.parse_args(argv)


def prepare_model(model):
    """fp16 everywhere the reference puts it (inference.py:15-22)."""
    from .autograd_4bit import Autograd4bitQuantLinear
    model.half()
    for _, m in model.named_modules():
        if isinstance(m, Autograd4bitQuantLinear):
            if m.is_v1_model:
                m.zeros = m.zeros.half()
            m.scales = m.scales.half()
            m.bias = m.bias.half()
    return model


def main(argv=None):
    """Returns (text, seconds)."""
    args = _parse(argv)
    from . import models
    from .amp_wrapper import AMPWrapper
    from .autograd_4bit import load_llama_model_4bit_low_ram
    if models.HAVE_PEFT:
        from .monkeypatch.peft_tuners_lora_monkey_patch import replace_peft_model_with_int4_lora_model
        replace_peft_model_with_int4_lora_model()

    model, tokenizer = load_llama_model_4bit_low_ram(args.config_path, args.model_path, groupsize=args.groupsize,
                                                      is_v1_model=args.v1)
    if args.lora is not None:
        from .finetune import LORA_TARGETS, load_adapter
        models.inject_lora_layers(model, target_modules=LORA_TARGETS, r=args.lora_r, lora_alpha=args.lora_alpha)
        print(load_adapter(model, args.lora), "adapter tensors loaded from", args.lora)
    print("Fitting 4bit scales and zeros to half")
    prepare_model(model)

    print("Apply AMP Wrapper ...")
    AMPWrapper(model).apply_generate()

    batch = tokenizer(args.prompt, return_tensors="pt", add_special_tokens=False)
    batch = {k: v.cuda() for k, v in batch.items()}
    options = dict(SAMPLING, max_new_tokens=args.max_new_tokens)
    if args.greedy:
        options.update(do_sample=False, temperature=None, top_p=None, top_k=None)
    start = time.time()
    with torch.no_grad():
        generated = model.generate(inputs=batch["input_ids"], **options)
    text = tokenizer.decode(generated["sequences"].cpu().tolist()[0])
    seconds = time.time() - start
    print(text)
    print(seconds)
    return text, seconds


if __name__ == "__main__":
    main()
