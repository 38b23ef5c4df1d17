"""Settings object of the LoRA finetune script, with the attribute names of the reference's
src/alpaca_lora_4bit/Finetune4bConfig.py:2-93 (its `finetune.py` reads them as `ft_config.<name>`).

Derived values follow the reference: `gradient_accumulation_steps = batch_size // mbatch_size` (`:64`), divided
again by the world size under DDP (`:85-86`); dropout forced to 0 with gradient checkpointing (`:70`);
`val_set_size` above 1 is a row count, otherwise a fraction (`:71`); `WORLD_SIZE` / `LOCAL_RANK` from the
environment decide `ddp` and `device_map` (`:81-84`).
"""
import os

_PLAIN_FIELDS = (
    "dataset", "ds_type", "lora_out_dir", "lora_apply_dir", "resume_checkpoint", "llama_q4_config_dir",
    "llama_q4_model", "mbatch_size", "batch_size", "epochs", "lr", "cutoff_len", "lora_r", "lora_alpha",
    "gradient_checkpointing", "gradient_checkpointing_ratio", "warmup_steps", "save_steps", "save_total_limit",
    "logging_steps", "checkpoint", "skip", "verbose", "txt_row_thd", "use_eos_token", "groupsize", "v1",
    "flash_attention", "xformers", "backend",
)

# sections of the printed summary: (title, attributes)
_SUMMARY = (
    ("config", ("dataset", "ds_type", "lora_out_dir", "lora_apply_dir", "llama_q4_config_dir", "llama_q4_model")),
    ("training", ("mbatch_size", "batch_size", "gradient_accumulation_steps", "epochs", "lr", "cutoff_len", "lora_r",
                  "lora_alpha", "lora_dropout", "val_set_size", "gradient_checkpointing",
                  "gradient_checkpointing_ratio", "warmup_steps", "save_steps", "save_total_limit", "logging_steps",
                  "checkpoint", "skip", "world_size", "ddp", "device_map", "groupsize", "v1", "backend")),
)


class Finetune4bConfig:
    """Config holder for 4-bit LLaMA LoRA finetuning; keyword arguments as in the reference (`:5-20`)."""

    def __init__(self, dataset, ds_type, lora_out_dir, lora_apply_dir, resume_checkpoint, llama_q4_config_dir,
                 llama_q4_model, mbatch_size, batch_size, epochs, lr, cutoff_len, lora_r, lora_alpha, lora_dropout,
                 val_set_size, gradient_checkpointing, gradient_checkpointing_ratio, warmup_steps, save_steps,
                 save_total_limit, logging_steps, checkpoint, skip, verbose, txt_row_thd, use_eos_token, groupsize,
                 v1, local_rank, flash_attention, xformers, backend):
        given = locals()
        for name in _PLAIN_FIELDS:
            setattr(self, name, given[name])
        self.lora_dropout = 0 if gradient_checkpointing else lora_dropout
        self.val_set_size = int(val_set_size) if val_set_size > 1.0 else float(val_set_size)
        self.world_size = int(os.environ.get("WORLD_SIZE", 1))
        self.local_rank = int(os.environ.get("LOCAL_RANK", local_rank))
        self.ddp = self.world_size != 1
        self.device_map = {"": self.local_rank} if self.ddp else "auto"
        self.gradient_accumulation_steps = batch_size // mbatch_size
        if self.ddp:
            self.gradient_accumulation_steps //= self.world_size

    def __str__(self) -> str:
        lines = ["", "Parameters:"]
        for title, names in _SUMMARY:
            lines.append(f"{title:-^20}")
            lines.extend(f"{n}={getattr(self, n)!r}" for n in names)
            lines.append("")
        return "\n".join(lines)
