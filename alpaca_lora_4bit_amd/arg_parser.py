"""Command line of the LoRA finetune script: the flags, defaults and positional `dataset` of the
reference's src/alpaca_lora_4bit/arg_parser.py:5-80, returned as a `Finetune4bConfig` by `get_config()`
(`:83-117`; its `finetune.py:23-24` calls that before anything else is imported).

`--backend` keeps its two spellings; both select the HIP kernels here (see `autograd_4bit.switch_backend_to`).
"""
import argparse
import os

from .Finetune4bConfig import Finetune4bConfig

# (group, flags, argparse keywords); help texts are generated from the defaults
_CONFIG, _TRAINING = "config", "training"
_OPTIONS = (
    (_CONFIG, ("--ds_type",), dict(choices=["txt", "alpaca", "gpt4all", "bluemoon"], default="alpaca",
                                   help="Dataset structure format")),
    (_CONFIG, ("--lora_out_dir",), dict(default="alpaca_lora", help="Directory to place new LoRA")),
    (_CONFIG, ("--lora_apply_dir",), dict(default=None, help="Directory of a LoRA to apply before training")),
    (_TRAINING, ("--resume_checkpoint",), dict(default=None, help="Resume training from this checkpoint")),
    (_CONFIG, ("--llama_q4_config_dir",), dict(default="./llama-13b-4bit/",
                                               help="Directory with config.json, tokenizer files, ...")),
    (_CONFIG, ("--llama_q4_model",), dict(default="./llama-13b-4bit.pt", help="Quantized model file or directory")),
    (_TRAINING, ("--mbatch_size",), dict(default=1, type=int, help="Micro-batch size")),
    (_TRAINING, ("--batch_size",), dict(default=2, type=int, help="Batch size")),
    (_TRAINING, ("--epochs",), dict(default=3, type=int, help="Epochs")),
    (_TRAINING, ("--lr",), dict(default=2e-4, type=float, help="Learning rate")),
    (_TRAINING, ("--cutoff_len",), dict(default=256, type=int, help="Maximum tokens per sample")),
    (_TRAINING, ("--lora_r",), dict(default=8, type=int, help="LoRA rank")),
    (_TRAINING, ("--lora_alpha",), dict(default=16, type=int, help="LoRA alpha")),
    (_TRAINING, ("--lora_dropout",), dict(default=0.05, type=float, help="LoRA dropout")),
    (_TRAINING, ("--grad_chckpt",), dict(action="store_true", help="Use gradient checkpointing")),
    (_TRAINING, ("--grad_chckpt_ratio",), dict(default=1, type=float, help="Share of decoder blocks to checkpoint")),
    (_TRAINING, ("--val_set_size",), dict(default=0.2, type=float, help="Validation set size (fraction or rows)")),
    (_TRAINING, ("--warmup_steps",), dict(default=50, type=int, help="Warm-up steps")),
    (_TRAINING, ("--save_steps",), dict(default=50, type=int, help="Steps between checkpoints")),
    (_TRAINING, ("--save_total_limit",), dict(default=3, type=int, help="Checkpoints kept")),
    (_TRAINING, ("--logging_steps",), dict(default=10, type=int, help="Steps between log lines")),
    (_TRAINING, ("-c", "--checkpoint"), dict(action="store_true", help="Produce a checkpoint instead of a LoRA")),
    (_TRAINING, ("--skip",), dict(action="store_true", help="Do not train (e.g. only re-save an existing LoRA)")),
    (_TRAINING, ("--verbose",), dict(action="store_true", help="Verbose training log")),
    (_TRAINING, ("--txt_row_thd",), dict(default=-1, type=int, help="Merge txt rows up to this many characters")),
    (_TRAINING, ("--use_eos_token",), dict(default=1, type=int, help="1: end samples with EOS, 0: pad to length")),
    (_TRAINING, ("--groupsize",), dict(default=-1, type=int, help="Group size of a v2 model")),
    (_TRAINING, ("--v1",), dict(action="store_true", help="The model uses the v1 layout")),
    (_TRAINING, ("--local_rank",), dict(default=0, type=int, help="Local rank under torch.distributed.launch")),
    (_TRAINING, ("--flash_attention",), dict(action="store_true", help="Use the flash-attention patch")),
    (_TRAINING, ("--xformers",), dict(action="store_true", help="Use the xformers attention patch")),
    (_TRAINING, ("--backend",), dict(default="cuda", type=str, help="Kernel backend name: cuda or triton")),
)

# argparse destination -> Finetune4bConfig keyword where the two differ
_RENAMED = {"grad_chckpt": "gradient_checkpointing", "grad_chckpt_ratio": "gradient_checkpointing_ratio"}


def _build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(prog=os.path.basename(__file__), description="Produce LoRA in 4bit training",
                                     usage="%(prog)s [config] [training]\n\nAll arguments are optional")
    parser.add_argument("dataset", nargs="?", default="./dataset.json", help="Path to dataset file. Default: %(default)s")
    groups = {name: parser.add_argument_group(name) for name in (_CONFIG, _TRAINING)}
    for group, flags, kw in _OPTIONS:
        kw = dict(kw)
        kw["help"] = kw["help"] + ". Default: %(default)s"
        groups[group].add_argument(*flags, required=False, **kw)
    return parser


def parse_commandline(argv=None) -> dict:
    """Parsed options as a dict keyed by flag name (`sys.argv` when `argv` is None)."""
    return vars(_build_parser().parse_args(argv))


def get_config(argv=None) -> Finetune4bConfig:
    args = parse_commandline(argv)
    kwargs = {_RENAMED.get(k, k): v for k, v in args.items()}
    kwargs["use_eos_token"] = kwargs["use_eos_token"] != 0
    return Finetune4bConfig(**kwargs)
