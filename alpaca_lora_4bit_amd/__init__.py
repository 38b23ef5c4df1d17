"""MI355X-native 4-bit GPTQ dequant-matmul path with the alpaca_lora_4bit operator interface.

Sub-modules keep the reference's names so its callers read unchanged:
    autograd_4bit        Autograd4bitQuantLinear, AutogradMatmul4bit, switch_backend_to, ...
    matmul_utils_4bit    matmul4bit, _matmul4bit_v2, _matmul4bit_v2_recons and the module knobs
    quant_hip            tensor-level mirror of the reference's quant_cuda extension module
    models               Linear4bitLt, GPTQLoraModel
    monkeypatch.peft_tuners_lora_monkey_patch   replace_peft_model_with_int4_lora_model
    arg_parser, Finetune4bConfig, train_data, gradient_checkpointing   what the finetune script imports
    finetune, inference  the reference's two top-level scripts as runnable modules (python -m ...)

`install_as_alpaca_lora_4bit()` registers these modules under the reference's package name so
that `from alpaca_lora_4bit import autograd_4bit` in an unmodified caller resolves here.

The arithmetic lives in libq4gptq.so (hand-written gfx950 HIP, C ABI in include/q4_gptq.h);
there is no CPU or pure-torch fallback: importing `quant_hip` without the built library raises.
"""
import importlib
import sys

__version__ = "0.1.0"

_ALIASED = ("autograd_4bit", "matmul_utils_4bit", "quant_hip", "models", "amp_wrapper", "model_attn_mlp_patch",
            "loaders", "arg_parser", "Finetune4bConfig", "train_data", "gradient_checkpointing", "monkeypatch",
            "monkeypatch.peft_tuners_lora_monkey_patch")


def install_as_alpaca_lora_4bit(name: str = "alpaca_lora_4bit") -> None:
    """Make `import alpaca_lora_4bit.<module>` resolve to this package's modules."""
    pkg = sys.modules[__name__]
    sys.modules.setdefault(name, pkg)
    for sub in _ALIASED:
        mod = importlib.import_module(f"{__name__}.{sub}")
        sys.modules.setdefault(f"{name}.{sub}", mod)
    # the reference binds its extension as alpaca_lora_4bit.quant_cuda (matmul_utils_4bit.py:6)
    quant_hip = importlib.import_module(f"{__name__}.quant_hip")
    sys.modules.setdefault(f"{name}.quant_cuda", quant_hip)
    pkg.quant_cuda = quant_hip
