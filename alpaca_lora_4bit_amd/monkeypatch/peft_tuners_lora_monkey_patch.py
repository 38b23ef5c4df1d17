"""Installs the 4-bit LoRA layer into peft (interface of the reference's
src/alpaca_lora_4bit/monkeypatch/peft_tuners_lora_monkey_patch.py:1-9, written for peft 0.6)."""


def replace_peft_model_with_int4_lora_model():
    try:
        import peft.peft_model
        from peft import PeftType
        from peft.tuners.lora import LoraModel
    except ImportError as e:
        raise ImportError("replace_peft_model_with_int4_lora_model() needs peft (the reference pins peft==0.6.*); "
                          "without peft use alpaca_lora_4bit_amd.models.inject_lora_layers") from e
    from ..models import GPTQLoraModel
    peft.peft_model.PEFT_TYPE_TO_MODEL_MAPPING[PeftType.LORA] = GPTQLoraModel
    LoraModel._create_new_module = GPTQLoraModel._create_new_module
    LoraModel._replace_module = GPTQLoraModel._replace_module
    print('Replaced _create_new_module and _replace_module of peft LoraModel with the 4-bit versions')
