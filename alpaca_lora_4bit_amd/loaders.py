"""Checkpoint loaders: build a LLaMA skeleton on the meta device, swap every nn.Linear except lm_head
for an empty Autograd4bitQuantLinear and let accelerate stream the GPTQ state dict
(`<module>.qweight / qzeros / scales / g_idx / bias`, safetensors or torch `.pt`) into it.

Mirrors src/alpaca_lora_4bit/autograd_4bit.py:250-360 of the reference: same function names, arguments,
defaults and side effects (`model.seqlen`, `tokenizer.truncation_side = 'left'`), so finetune.py /
inference.py call them unchanged.  The layers they create run on the HIP kernels of this package.
"""
import logging
import time

import torch

from .autograd_4bit import (Autograd4bitQuantLinear, find_layers, make_quant_for_4bit_autograd, model_to_half)

log = logging.getLogger(__name__)

_NO_SPLIT = ["LlamaDecoderLayer"]


def _empty_quantized_llama(config_path, groupsize, is_v1_model, bits):
    """LlamaForCausalLM without weights whose Linear layers (lm_head excepted) are quantized stubs
    (autograd_4bit.py:257-266)."""
    import accelerate
    from transformers import LlamaConfig, LlamaForCausalLM
    with accelerate.init_empty_weights():
        config = LlamaConfig.from_pretrained(config_path)
        model = LlamaForCausalLM(config)
        model = model.eval()
        layers = find_layers(model)
        layers.pop('lm_head', None)
        make_quant_for_4bit_autograd(model, layers, groupsize=groupsize, is_v1_model=is_v1_model, bits=bits)
    return model


def _load_tokenizer(config_path, model=None):
    """LlamaTokenizer of the config directory, truncating on the left (autograd_4bit.py:279-283)."""
    from transformers import LlamaTokenizer
    try:
        tokenizer = LlamaTokenizer.from_pretrained(config_path)
    except Exception as first_error:                      # the reference retries on HFValidationError only
        if model is None:
            raise
        try:
            tokenizer = LlamaTokenizer.from_pretrained(model)
        except Exception:
            raise first_error
    tokenizer.truncation_side = 'left'
    return tokenizer


def _half_quant_buffers(model, also=()):
    """scales / bias (and v1 zeros) of every quantized layer to fp16 (autograd_4bit.py:336-342)."""
    kinds = (Autograd4bitQuantLinear,) + tuple(also)
    for _, m in model.named_modules():
        if isinstance(m, kinds):
            if m.is_v1_model:
                m.zeros = m.zeros.half()
            m.scales = m.scales.half()
            m.bias = m.bias.half()


def load_llama_model_4bit_low_ram(config_path, model_path, groupsize=-1, half=False, device_map="auto", seqlen=2048,
                                  is_v1_model=False, bits=4):
    """autograd_4bit.py:250-287.  Returns (model, tokenizer)."""
    import accelerate
    log.info("Loading Model ...")
    t0 = time.time()
    model = _empty_quantized_llama(config_path, groupsize, is_v1_model, bits)
    model = accelerate.load_checkpoint_and_dispatch(model=model, checkpoint=model_path, device_map=device_map,
                                                    no_split_module_classes=_NO_SPLIT)
    model.seqlen = seqlen
    if half:
        model_to_half(model)
    tokenizer = _load_tokenizer(config_path, model)
    log.info("Loaded the model in %.2f seconds.", time.time() - t0)
    return model, tokenizer


def load_llama_model_4bit_low_ram_and_offload(config_path, model_path, lora_path=None, groupsize=-1, seqlen=2048,
                                              max_memory=None, is_v1_model=False, bits=4):
    """autograd_4bit.py:289-358: load on the CPU, optionally attach a LoRA adapter, cast the quantization
    buffers to fp16, then let accelerate place the decoder layers under `max_memory` with the rest
    offloaded to host memory.  Returns (model, tokenizer)."""
    import accelerate
    if max_memory is None:
        max_memory = {0: '24Gib', 'cpu': '48Gib'}
    log.info("Loading Model ...")
    t0 = time.time()
    model = _empty_quantized_llama(config_path, groupsize, is_v1_model, bits)
    accelerate.load_checkpoint_in_model(model, checkpoint=model_path, device_map={'': 'cpu'})

    lora_layer_types = ()
    if lora_path is not None:
        from .monkeypatch.peft_tuners_lora_monkey_patch import replace_peft_model_with_int4_lora_model
        replace_peft_model_with_int4_lora_model()
        try:
            from peft import PeftModel
        except ImportError as e:
            raise ImportError("lora_path was given but peft is not installed: PeftModel.from_pretrained is what "
                              "reads an adapter directory (autograd_4bit.py:321-325)") from e
        from .models import Linear4bitLt
        lora_layer_types = (Linear4bitLt,)
        model = PeftModel.from_pretrained(model, lora_path, device_map={'': 'cpu'}, torch_dtype=torch.float32,
                                          is_trainable=True)
        log.info("%s Lora Applied.", lora_path)

    model.seqlen = seqlen
    _half_quant_buffers(model, also=lora_layer_types)

    device_map = accelerate.infer_auto_device_map(model, max_memory=max_memory, no_split_module_classes=_NO_SPLIT)
    model = accelerate.dispatch_model(model, device_map=device_map, offload_buffers=True, main_device=0)
    if torch.cuda.is_available():
        torch.cuda.empty_cache()
        log.info("Total %.2f MiB VRAM used.", torch.cuda.memory_allocated() / 1024 / 1024)
    tokenizer = _load_tokenizer(config_path)
    log.info("Loaded the model in %.2f seconds.", time.time() - t0)
    return model, tokenizer


load_llama_model_4bit_low_ram_and_offload_to_cpu = load_llama_model_4bit_low_ram_and_offload
