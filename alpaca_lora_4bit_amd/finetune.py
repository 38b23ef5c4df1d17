"""LoRA finetuning of a 4-bit GPTQ LLaMA: the flow of the reference's top-level finetune.py:22-198 as a module,

    python -m alpaca_lora_4bit_amd.finetune ./data.txt --ds_type txt --llama_q4_config_dir ./llama-7b-4bit/ \\
        --llama_q4_model ./llama-7b-4bit/model.safetensors --groupsize 128

with the same command line (`arg_parser`) and the same order of steps: patch peft, pick the backend, load the packed
model, add LoRA to q_proj / v_proj, halve the scales, read the dataset, optionally checkpoint the decoder blocks,
train with `transformers.Trainer` under fp16 autocast, save the adapter.

Two optional dependencies of the reference are optional here as well: with peft installed the adapter is created
and saved by peft (`get_peft_model`, `PeftModel.from_pretrained`, `save_pretrained`, finetune.py:75-95,194);
without it `models.inject_lora_layers` builds the same `Linear4bitLt` layers and the adapter is written in peft's
file layout (`adapter_config.json` + `adapter_model.safetensors`, keys `base_model.model.<module>.lora_A.weight`)
so that peft can read it later.  wandb is used when importable (finetune.py:183), skipped otherwise.
The flash-attention / xformers attention patches of the reference are not part of this package; their flags are
accepted and ignored with a note.
"""
import json
import os

import torch

LORA_TARGETS = ["q_proj", "v_proj"]                  # finetune.py:78


def _adapter_state(model):
    """LoRA tensors under the names peft gives them in adapter_model.safetensors."""
    state = {}
    for name, module in model.named_modules():
        if "Linear4bitLt" not in str(type(module)):
            continue
        for part in ("lora_A", "lora_B"):
            for adapter, layer in getattr(module, part).items():
                if adapter == "default":
                    state[f"base_model.model.{name}.{part}.weight"] = layer.weight.detach().cpu().contiguous()
    return state


def save_adapter(model, out_dir, ft_config):
    """peft's `save_pretrained` when the model is a PeftModel, otherwise the same two files written by hand."""
    os.makedirs(out_dir, exist_ok=True)
    if hasattr(model, "peft_config"):
        model.save_pretrained(out_dir)
        return
    from safetensors.torch import save_file
    save_file(_adapter_state(model), os.path.join(out_dir, "adapter_model.safetensors"))
    with open(os.path.join(out_dir, "adapter_config.json"), "w") as fh:
        json.dump({"peft_type": "LORA", "task_type": "CAUSAL_LM", "r": ft_config.lora_r,
                   "lora_alpha": ft_config.lora_alpha, "lora_dropout": ft_config.lora_dropout, "bias": "none",
                   "target_modules": LORA_TARGETS, "fan_in_fan_out": False, "inference_mode": True,
                   "base_model_name_or_path": ft_config.llama_q4_config_dir}, fh, indent=2)


def load_adapter(model, adapter_dir):
    """Reads an adapter written by `save_adapter` (or by peft) into the Linear4bitLt layers of `model`."""
    from safetensors.torch import load_file
    state = load_file(os.path.join(adapter_dir, "adapter_model.safetensors"))
    modules = dict(model.named_modules())
    loaded = 0
    for key, tensor in state.items():
        path = key[len("base_model.model."):] if key.startswith("base_model.model.") else key
        mod_name, part, _ = path.rsplit(".", 2)
        layer = getattr(modules[mod_name], part)["default"]
        with torch.no_grad():
            layer.weight.copy_(tensor.to(layer.weight.dtype))
        loaded += 1
    return loaded


def _add_lora(model, ft_config):
    from . import models
    if models.HAVE_PEFT:
        from peft import LoraConfig, PeftModel, get_peft_model
        if ft_config.lora_apply_dir is None:
            lora_config = LoraConfig(r=ft_config.lora_r, lora_alpha=ft_config.lora_alpha, target_modules=LORA_TARGETS,
                                     lora_dropout=ft_config.lora_dropout, bias="none", task_type="CAUSAL_LM")
            return get_peft_model(model, lora_config)
        device_map = {"": 0} if (ft_config.ddp or torch.cuda.device_count() <= 1) else "auto"
        print("Device map for lora:", device_map)
        model = PeftModel.from_pretrained(model, ft_config.lora_apply_dir, device_map=device_map,
                                          torch_dtype=torch.float32, is_trainable=True)
        print(ft_config.lora_apply_dir, "loaded")
        return model
    layers = models.inject_lora_layers(model, target_modules=LORA_TARGETS, r=ft_config.lora_r,
                                       lora_alpha=ft_config.lora_alpha, lora_dropout=ft_config.lora_dropout)
    print(f"LoRA added to {len(layers)} layers (peft not installed: built-in injection)")
    if ft_config.lora_apply_dir is not None:
        print(load_adapter(model, ft_config.lora_apply_dir), "adapter tensors loaded from", ft_config.lora_apply_dir)
    return model


def _pick_reader(ft_config, tokenizer):
    from . import train_data
    readers = {"txt": train_data.TrainTxt, "alpaca": train_data.TrainSAD, "gpt4all": train_data.TrainGPT4All,
               "bluemoon": train_data.TrainBlueMoon}
    if ft_config.ds_type not in readers:
        raise NotImplementedError("ERROR: Unknown dataset format")
    return readers[ft_config.ds_type](ft_config.dataset, ft_config.val_set_size, tokenizer, ft_config.cutoff_len)


def _train(model, tokenizer, data, ft_config):
    import transformers
    if ft_config.val_set_size > 0 and data.val_data is not None:
        # ten evaluations over the run, but not more often than the log lines (finetune.py:140-148)
        eval_steps = max(ft_config.logging_steps,
                         (len(data.train_data) + len(data.val_data)) // (10 * ft_config.mbatch_size))
        print(f"Run eval every {eval_steps} steps")
    else:
        eval_steps = 0
    keeps_adapter_checkpoints = hasattr(model, "peft_config")
    if not keeps_adapter_checkpoints:
        print("peft not installed: intermediate checkpoints are switched off, the adapter is saved at the end")
    args = transformers.TrainingArguments(
        per_device_train_batch_size=ft_config.mbatch_size,
        gradient_accumulation_steps=ft_config.gradient_accumulation_steps,
        warmup_steps=ft_config.warmup_steps,
        optim="adamw_torch",
        num_train_epochs=ft_config.epochs,
        learning_rate=ft_config.lr,
        fp16=True,
        logging_steps=ft_config.logging_steps,
        eval_strategy="steps" if eval_steps else "no",
        eval_steps=eval_steps or None,
        save_strategy="steps" if keeps_adapter_checkpoints else "no",
        save_steps=ft_config.save_steps,
        output_dir=ft_config.lora_out_dir,
        save_total_limit=ft_config.save_total_limit,
        load_best_model_at_end=False,
        ddp_find_unused_parameters=False if ft_config.ddp else None,
        report_to="none",
    )
    trainer = transformers.Trainer(
        model=model, train_dataset=data.train_data, eval_dataset=data.val_data if eval_steps else None, args=args,
        data_collator=transformers.DataCollatorForLanguageModeling(tokenizer, mlm=False))
    model.config.use_cache = False
    if ft_config.verbose:
        transformers.logging.set_verbosity_info()
    try:
        import wandb
        run = wandb.init(project="alpaca_lora_4bit")
    except ImportError:
        run = None
    try:
        if ft_config.resume_checkpoint:
            print("Resuming from {} ...".format(ft_config.resume_checkpoint))
            result = trainer.train(resume_from_checkpoint=ft_config.resume_checkpoint)
        else:
            result = trainer.train()
    finally:
        if run is not None:
            run.finish()
    print("Train completed.")
    return trainer, result


def main(argv=None):
    """Runs the whole flow; returns (model, tokenizer, trainer or None)."""
    from .arg_parser import get_config
    ft_config = get_config(argv)

    from . import models
    if models.HAVE_PEFT:
        from .monkeypatch.peft_tuners_lora_monkey_patch import replace_peft_model_with_int4_lora_model
        replace_peft_model_with_int4_lora_model()
    if ft_config.flash_attention or ft_config.xformers:
        print("note: the flash-attention / xformers patches are not provided here; the model's own attention runs")

    from . import autograd_4bit
    autograd_4bit.switch_backend_to("triton" if ft_config.backend.lower() == "triton" else "cuda")

    if ft_config.local_rank == 0:
        print(f"{ft_config}\n")
    if ft_config.gradient_checkpointing:
        print("Disable Dropout.")
    if ft_config.mbatch_size > ft_config.batch_size:
        raise Exception("batch_size need to be larger than mbatch_size.")

    model, tokenizer = autograd_4bit.load_llama_model_4bit_low_ram(
        ft_config.llama_q4_config_dir, ft_config.llama_q4_model, device_map=ft_config.device_map,
        groupsize=ft_config.groupsize, is_v1_model=ft_config.v1)
    model = _add_lora(model, ft_config)

    print("Fitting 4bit scales and zeros to half")
    for _, m in model.named_modules():
        if "Autograd4bitQuantLinear" in str(type(m)) or "Linear4bitLt" in str(type(m)):
            if getattr(m, "is_v1_model", False):
                m.zeros = m.zeros.half()
            m.scales = m.scales.half()
    tokenizer.pad_token_id = 0

    trainer = None
    if not ft_config.skip:
        data = _pick_reader(ft_config, tokenizer)
        data.prepare_data(thd=ft_config.txt_row_thd, use_eos_token=ft_config.use_eos_token)
        if ft_config.gradient_checkpointing:
            print("Applying gradient checkpointing ...")
            from .gradient_checkpointing import apply_gradient_checkpointing
            apply_gradient_checkpointing(model, checkpoint_ratio=ft_config.gradient_checkpointing_ratio)
        if not ft_config.ddp and torch.cuda.device_count() > 1:
            model.is_parallelizable = True           # keeps Trainer from wrapping the model in DataParallel
            model.model_parallel = True
        trainer, _ = _train(model, tokenizer, data, ft_config)

    save_adapter(model, ft_config.lora_out_dir, ft_config)
    if ft_config.checkpoint:
        print("Warning: Merge model + LoRA and save the whole checkpoint not implemented yet.")
    print("Model Saved.")
    return model, tokenizer, trainer


if __name__ == "__main__":
    main()
