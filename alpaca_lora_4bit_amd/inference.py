"""Text generation with a 4-bit GPTQ LLaMA: the flow of the reference's top-level inference.py:1-49 as a module,

    python -m alpaca_lora_4bit_amd.inference ./llama-7b-4bit/ ./llama-7b-4bit/model.safetensors --groupsize 128 \\
        --prompt "I think the meaning of life is"

Steps as in the reference: load the packed model, `model.half()` and halve `scales` / `bias` (v1: `zeros`) of every
4-bit layer (`:15-22`), wrap `generate` in autocast (`:24-27`), sample with the reference's settings (`:33-44`:
temperature 0.9, top-p 0.95, top-k 40, repetition penalty 1.1, 20 new tokens), print the text and the seconds taken.
`--lora` applies an adapter directory written by `alpaca_lora_4bit_amd.finetune` (or by peft) first.

Two additions for decode speed, both off by default: `--fuse` gives q/k/v one grouped launch on their own tensors and
runs the MLP decode step (gate, up, silu * up, down) as one launch, adapters included
(model_attn_mlp_patch.make_quant_attn / make_fused_mlp, which the reference's model server calls, server/server.py:100-113),
and `--hip_graph` captures the one-token step once as a HIP graph and replays it per token, which removes the host
time of the ~1000 small launches a decoder step consists of; the choice of the next token (argmax with `--greedy`,
otherwise the reference's sampling settings) runs eagerly between two replays.
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
    p.add_argument("--fuse", action="store_true", help="one launch for q+k+v and one for gate+up")
    p.add_argument("--hip_graph", action="store_true", help="decode with the token step replayed as a HIP graph")
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


def _token_picker(sampling):
    """Returns pick(ids_so_far, logits) -> next token [1, 1].  `sampling` None: argmax.  Otherwise a dict with the
    reference's settings (inference.py:33-44: repetition_penalty, temperature, top_k, top_p) applied through
    transformers' own logits processors in the order `generate` applies them, then one multinomial draw."""
    if sampling is None:
        return lambda ids, logits: logits.argmax(-1, keepdim=True)
    from transformers import (LogitsProcessorList, RepetitionPenaltyLogitsProcessor, TemperatureLogitsWarper,
                              TopKLogitsWarper, TopPLogitsWarper)
    procs = LogitsProcessorList()
    if sampling.get("repetition_penalty", 1.0) != 1.0:
        procs.append(RepetitionPenaltyLogitsProcessor(penalty=sampling["repetition_penalty"]))
    if sampling.get("temperature", 1.0) != 1.0:
        procs.append(TemperatureLogitsWarper(sampling["temperature"]))
    if sampling.get("top_k"):
        procs.append(TopKLogitsWarper(top_k=sampling["top_k"]))
    if sampling.get("top_p", 1.0) < 1.0:
        procs.append(TopPLogitsWarper(top_p=sampling["top_p"]))

    def pick(ids, logits):
        scores = procs(ids, logits.float())
        return torch.multinomial(torch.softmax(scores, dim=-1), num_samples=1)
    return pick


def generate_graph(model, input_ids, max_new_tokens, eos_token_id=None, sampling=None, use_graph=True):
    """Decoding of one sequence with the model's one-token forward captured once as a HIP graph and replayed for
    every further token: eager prefill into a static KV cache, the second token from one eager step (the warm-up
    that graph capture wants: every lazy allocation and per-layer check of the kernels' host side happens there),
    then replays.  Token id and position live in device buffers that the replays read; the choice of the next
    token (argmax, or the logits processors + multinomial of `sampling`) runs eagerly between two replays.
    `use_graph=False` runs the same loop without capture.  Returns the ids [1, prompt + new] like `generate`;
    stops early at `eos_token_id`."""
    from transformers import StaticCache
    dev = input_ids.device
    prompt = input_ids.shape[1]
    pick = _token_picker(sampling)
    with torch.no_grad():
        cache = StaticCache(config=model.config, max_cache_len=prompt + max_new_tokens)
        out = model(input_ids=input_ids, past_key_values=cache, use_cache=True,
                    cache_position=torch.arange(prompt, device=dev))
        ids = input_ids
        tok_buf = torch.empty((1, 1), dtype=input_ids.dtype, device=dev)
        pos_buf = torch.tensor([prompt - 1], device=dev)

        def advance(logits):
            nonlocal ids
            nxt = pick(ids, logits)
            tok_buf.copy_(nxt)
            pos_buf.add_(1)
            ids = torch.cat([ids, nxt], dim=1)
            return eos_token_id is not None and int(nxt[0, 0]) == eos_token_id

        def step():
            o = model(input_ids=tok_buf, past_key_values=cache, use_cache=True, cache_position=pos_buf)
            return o.logits[:, -1]

        done = advance(out.logits[:, -1])
        if not done and max_new_tokens > 1:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                logits = step()
            torch.cuda.current_stream().wait_stream(side)
            done = advance(logits)
            remaining = max_new_tokens - 2
            if not done and remaining > 0:
                if use_graph:
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph):
                        logits = step()
                for _ in range(remaining):
                    if use_graph:
                        graph.replay()
                    else:
                        logits = step()
                    if advance(logits):
                        break
    return ids


def greedy_generate_graph(model, input_ids, max_new_tokens, eos_token_id=None):
    """`generate_graph` with argmax decoding."""
    return generate_graph(model, input_ids, max_new_tokens, eos_token_id=eos_token_id)


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

    if args.fuse:
        from .model_attn_mlp_patch import make_fused_mlp, make_quant_attn
        print("Fused", make_quant_attn(model), "attention blocks and", make_fused_mlp(model), "MLP blocks")

    print("Apply AMP Wrapper ...")
    AMPWrapper(model).apply_generate()

    batch = tokenizer(args.prompt, return_tensors="pt", add_special_tokens=False)
    batch = {k: v.cuda() for k, v in batch.items()}
    options = dict(SAMPLING, max_new_tokens=args.max_new_tokens)
    if args.greedy:
        options.update(do_sample=False, temperature=None, top_p=None, top_k=None)
    start = time.time()
    if args.hip_graph:
        sampling = None if args.greedy else {k: SAMPLING[k] for k in ("repetition_penalty", "temperature", "top_k", "top_p")}
        with torch.amp.autocast(device_type="cuda"):
            sequences = generate_graph(model, batch["input_ids"], args.max_new_tokens,
                                       eos_token_id=getattr(tokenizer, "eos_token_id", None), sampling=sampling)
    else:
        with torch.no_grad():
            sequences = model.generate(inputs=batch["input_ids"], **options)["sequences"]
    text = tokenizer.decode(sequences.cpu().tolist()[0])
    seconds = time.time() - start
    print(text)
    print(seconds)
    return text, seconds


if __name__ == "__main__":
    main()
