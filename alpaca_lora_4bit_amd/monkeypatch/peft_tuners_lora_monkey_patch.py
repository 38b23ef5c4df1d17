"""Makes peft build `Linear4bitLt` layers for 4-bit targets: the entry point
`replace_peft_model_with_int4_lora_model()` of the reference's
src/alpaca_lora_4bit/monkeypatch/peft_tuners_lora_monkey_patch.py:1-9 (written for peft 0.6).

Two hooks of peft's `LoraModel` are redirected to `models.GPTQLoraModel` and the LORA entry of peft's
type-to-model table is pointed at it, so both `get_peft_model` and `PeftModel.from_pretrained` take the 4-bit
route.  Calling it twice is harmless; `restore_peft_lora_model()` puts peft's own objects back (useful in tests
and notebooks, the reference has no such call).
"""

_HOOKS = ("_create_new_module", "_replace_module")
_saved = {}


def _peft_objects():
    try:
        import peft.peft_model as peft_model
        from peft import PeftType
        from peft.tuners.lora import LoraModel
    except ImportError as e:
        raise ImportError("replace_peft_model_with_int4_lora_model() needs peft (the reference pins peft==0.6.*); "
                          "without peft use alpaca_lora_4bit_amd.models.inject_lora_layers") from e
    return peft_model.PEFT_TYPE_TO_MODEL_MAPPING, PeftType.LORA, LoraModel


def replace_peft_model_with_int4_lora_model():
    table, lora_key, lora_model = _peft_objects()
    from ..models import GPTQLoraModel
    if not _saved:
        _saved["table_entry"] = table.get(lora_key)
        for hook in _HOOKS:
            _saved[hook] = lora_model.__dict__.get(hook)
    table[lora_key] = GPTQLoraModel
    for hook in _HOOKS:
        setattr(lora_model, hook, staticmethod(getattr(GPTQLoraModel, hook)))
    print("peft LoraModel now builds Linear4bitLt for 4-bit layers (" + ", ".join(_HOOKS) + " replaced)")


def restore_peft_lora_model():
    """Undo replace_peft_model_with_int4_lora_model()."""
    if not _saved:
        return
    table, lora_key, lora_model = _peft_objects()
    table[lora_key] = _saved.pop("table_entry")
    for hook in _HOOKS:
        original = _saved.pop(hook)
        if original is not None:
            setattr(lora_model, hook, original)
