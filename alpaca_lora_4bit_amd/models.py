"""LoRA on top of the 4-bit linear: `Linear4bitLt` and `GPTQLoraModel` with the interface of the
reference's src/alpaca_lora_4bit/models.py:13-163 (written against peft 0.6).

When peft is importable its `LoraLayer` / `LoraModel` are the base classes, exactly as in the
reference.  When it is not, a small stand-in `LoraLayer` with the same attribute names
(`r, lora_alpha, scaling, lora_dropout, lora_A, lora_B, active_adapters, disable_adapters,
update_layer, set_adapter`) keeps `Linear4bitLt` usable on its own.  The stand-in follows
peft 0.6's documented behaviour (A: Kaiming-uniform with a=sqrt(5), B: zeros, scaling =
lora_alpha / r); peft itself could not be imported where this was written, so equality with
peft's internals is not verified -- the adapter arithmetic (models.py:58-66) is.
"""
import math

import torch
import torch.nn as nn

from . import autograd_4bit
from .autograd_4bit import Autograd4bitQuantLinear

try:  # pragma: no cover - depends on the environment
    from peft.tuners import lora as _peft_lora
    from peft.tuners.lora import LoraLayer
    HAVE_PEFT = True
except ImportError:
    _peft_lora = None
    HAVE_PEFT = False

    class LoraLayer:
        """Minimal stand-in for peft.tuners.lora.LoraLayer (see the module docstring)."""

        adapter_layer_names = ("lora_A", "lora_B")

        def __init__(self, in_features: int, out_features: int, **kwargs):
            self.r = {}
            self.lora_alpha = {}
            self.scaling = {}
            self.lora_dropout = nn.ModuleDict({})
            self.lora_A = nn.ModuleDict({})
            self.lora_B = nn.ModuleDict({})
            self._disable_adapters = False
            self._active_adapter = "default"
            self.merged_adapters = []
            self.in_features = in_features
            self.out_features = out_features
            self.kwargs = kwargs

        @property
        def disable_adapters(self):
            return self._disable_adapters

        @property
        def active_adapters(self):
            a = self._active_adapter
            return [a] if isinstance(a, str) else list(a)

        @property
        def active_adapter(self):
            return self._active_adapter

        def enable_adapters(self, enabled: bool):
            self._disable_adapters = not enabled

        def set_adapter(self, adapter_names):
            if isinstance(adapter_names, str):
                adapter_names = [adapter_names]
            for layer_name in self.adapter_layer_names:
                for key, layer in getattr(self, layer_name).items():
                    layer.requires_grad_(key in adapter_names)
            self._active_adapter = adapter_names

        def update_layer(self, adapter_name, r, lora_alpha, lora_dropout, init_lora_weights):
            if r <= 0:
                raise ValueError(f"`r` should be a positive integer value but the value passed is {r}")
            self.r[adapter_name] = r
            self.lora_alpha[adapter_name] = lora_alpha
            self.lora_dropout[adapter_name] = nn.Dropout(p=lora_dropout) if lora_dropout > 0.0 else nn.Identity()
            self.lora_A[adapter_name] = nn.Linear(self.in_features, r, bias=False)
            self.lora_B[adapter_name] = nn.Linear(r, self.out_features, bias=False)
            self.scaling[adapter_name] = lora_alpha / r
            if init_lora_weights:
                nn.init.kaiming_uniform_(self.lora_A[adapter_name].weight, a=math.sqrt(5))
                nn.init.zeros_(self.lora_B[adapter_name].weight)
            weight = getattr(self, "weight", None)
            if weight is not None:
                for name in self.adapter_layer_names:
                    getattr(self, name)[adapter_name].to(weight.device)
            self.set_adapter(self.active_adapters)


# Use the fused GEMM (adapter folded into the main kernel) whenever the case allows it.
fuse_lora = True


class Linear4bitLt(Autograd4bitQuantLinear, LoraLayer):
    """4-bit linear + LoRA adapters (models.py:13-76)."""

    def __init__(self, adapter_name, in_features, out_features, groupsize: int = -1, is_v1_model: bool = False,
                 r: int = 0, lora_alpha: int = 1, lora_dropout: float = 0.0, **kwargs):
        Autograd4bitQuantLinear.__init__(self, in_features, out_features, groupsize, is_v1_model)
        LoraLayer.__init__(self, in_features=in_features, out_features=out_features)

        # the quantized base weights are frozen (models.py:37-45)
        for name in ('qweight', 'scales', 'bias') + (('zeros',) if self.is_v1_model else ('qzeros', 'g_idx')):
            getattr(self, name).requires_grad = False

        init_lora_weights = kwargs.pop("init_lora_weights", True)
        self.update_layer(adapter_name, r, lora_alpha, lora_dropout, init_lora_weights)
        self.set_adapter(adapter_names=[adapter_name])

    # ---- fused path --------------------------------------------------------------------
    def _fusable_adapter(self, x):
        """Name of the single adapter the fused kernel can take for this call, else None."""
        if not fuse_lora or self.is_v1_model or self.bits != 4 or not x.is_cuda:
            return None
        if autograd_4bit.backend != 'cuda':
            return None
        active = [a for a in self.active_adapters if a in self.lora_A.keys()]
        if len(active) != 1:
            return None
        name = active[0]
        r = self.lora_A[name].weight.shape[0]
        if r % 8 != 0 or not (8 <= r <= 64):
            return None
        if self._dropout_p(name) >= 1.0 or (self._dropout_p(name) > 0.0 and torch.cuda.is_current_stream_capturing()):
            return None                                   # the mask's seed is a launch argument: a replayed graph would repeat it
        rows = x.numel() // x.shape[-1]
        if rows <= autograd_4bit.quant_hip.MAX_GEMV_ROWS:
            return None
        if self.in_features % 128 or self.out_features % 128:
            return None
        if not (torch.is_autocast_enabled('cuda') or x.dtype == torch.float16):
            return None
        return name

    def _dropout_p(self, name):
        """Probability of the adapter's dropout as it applies to this call (0 in eval mode / without dropout)."""
        drop = self.lora_dropout[name]
        if isinstance(drop, nn.Dropout) and drop.p > 0.0 and self.training:
            return float(drop.p)
        return 0.0

    def _decode_adapter(self, x):
        """Name of the single adapter for the short no-grad path (a handful of rows, eval mode), else None."""
        if torch.is_grad_enabled() or not fuse_lora or not x.is_cuda or self.bits != 4:
            return None
        if x.numel() // x.shape[-1] > autograd_4bit.quant_hip.MAX_GEMV_ROWS:
            return None
        active = [a for a in self.active_adapters if a in self.lora_A.keys()]
        if len(active) != 1:
            return None
        name = active[0]
        r = self.lora_A[name].weight.shape[0]
        drop = self.lora_dropout[name]
        if r < 1 or r > 64 or self.in_features % 32 or (isinstance(drop, nn.Dropout) and drop.p > 0.0 and self.training):
            return None
        return name

    def _half_lora_b(self, name):
        """fp16 [r, N] copy of lora_B.weight for the rank-r update, rebuilt when the parameter changes."""
        w = self.lora_B[name].weight
        key = (w._version, w.data_ptr(), w.dtype)
        cached = self.__dict__.get("_q4_lora_b16")
        if cached is None or cached[0] != key:
            cached = (key, w.detach().t().to(torch.float16).contiguous())
            self.__dict__["_q4_lora_b16"] = cached
        return cached[1]

    def forward(self, x: torch.Tensor):
        if not self.disable_adapters:
            name = self._decode_adapter(x)
            if name is not None:
                # decode: base product (GEMV), x @ A^T with the adapter read in place, one rank-r update in place:
                # three launches instead of the seven of the composition below, same values up to fp16 rounding
                result = Autograd4bitQuantLinear.forward(self, x)
                xa = autograd_4bit.quant_hip.lora_down(x.reshape(-1, x.shape[-1]).to(torch.float16).contiguous(),
                                                       self.lora_A[name].weight)
                out2 = result.view(-1, result.shape[-1])
                if out2.dtype == torch.float16:
                    out2.addmm_(xa, self._half_lora_b(name), alpha=float(self.scaling[name]))
                else:
                    out2.add_((xa @ self._half_lora_b(name)).to(out2.dtype), alpha=float(self.scaling[name]))
                return result
            name = self._fusable_adapter(x)
            if name is not None:
                group = self.__dict__.get('_q4_group')
                if group is not None:
                    out = group.run_gemm(self, x)            # one grouped launch for all members, adapters included
                    if out is not None:
                        return out
                bias = None
                if not self.disable_bias and not autograd_4bit._is_all_zero(self.bias):
                    bias = self.bias if self.bias.dtype == torch.float16 else self.bias.half()
                # dropout(x) in front of lora_A (models.py:63-66) stays inside the fused kernels: a counter-based mask
                # keyed by a seed drawn here from torch's CPU generator (so torch.manual_seed and the RNG state
                # that checkpointing restores for its recomputation reproduce it)
                drop_p = self._dropout_p(name)
                drop_seed = int(torch.randint(0, 2 ** 62, (1,)).item()) if drop_p > 0.0 else 0
                return autograd_4bit.AutogradMatmul4bitLora.apply(
                    x, self.qweight, self.scales, self.qzeros, self.g_idx, bias,
                    self.lora_A[name].weight, self.lora_B[name].weight, float(self.scaling[name]), self.groupsize,
                    drop_p, drop_seed)

        # reference composition (models.py:51-69)
        result = super().forward(x)
        if self.disable_adapters:
            return result
        previous_dtype = result.dtype
        for active_adapter in self.active_adapters:
            if active_adapter not in self.lora_A.keys():
                continue
            lora_A = self.lora_A[active_adapter]
            lora_B = self.lora_B[active_adapter]
            dropout = self.lora_dropout[active_adapter]
            scaling = self.scaling[active_adapter]
            x = x.to(lora_A.weight.dtype)
            result = result + (lora_B(lora_A(dropout(x))) * scaling).to(result.dtype)
        return result.to(previous_dtype)

    @property
    def weight(self):
        """Device/dtype carrier so that peft's update_layer moves the adapter weights to the
        GPU without changing their dtype (models.py:71-76: dtype is the int32 of qweight)."""
        qweight = self.qweight

        class WeightDeviceClass:
            device = qweight.device
            dtype = qweight.dtype
        return WeightDeviceClass()


def _share_quant_tensors(new_module, child):
    """models.py:119-127: the replacement shares the packed tensors with the layer it replaces."""
    new_module.qweight = child.qweight
    new_module.scales = child.scales
    if child.is_v1_model:
        new_module.zeros = child.zeros
    else:
        new_module.qzeros = child.qzeros
        new_module.g_idx = child.g_idx
    new_module.bias = child.bias


def _move_adapters(new_module, device):
    for name, module in new_module.named_modules():
        if "lora_" in name or "ranknum" in name:
            module.to(device)


if HAVE_PEFT:  # pragma: no cover - peft is not available where the tests run
    # peft's own hooks, taken before replace_peft_model_with_int4_lora_model() redirects them: every target that is
    # not a 4-bit layer is handed on to them unchanged
    _peft_create_new_module = _peft_lora.LoraModel.__dict__["_create_new_module"].__func__
    _peft_replace_module = _peft_lora.LoraModel.__dict__["_replace_module"]
    _peft_replace_module = getattr(_peft_replace_module, "__func__", _peft_replace_module)

    class GPTQLoraModel(_peft_lora.LoraModel):
        """peft LoraModel that builds Linear4bitLt for 4-bit targets (models.py:79-163)."""

        @staticmethod
        def _create_new_module(lora_config, adapter_name, target, **kwargs):
            if isinstance(target, Autograd4bitQuantLinear):
                bias = kwargs.pop("bias", False)
                return Linear4bitLt(adapter_name, target.in_features, target.out_features, target.groupsize,
                                    target.is_v1_model, bias=bias, **kwargs)
            return _peft_create_new_module(lora_config, adapter_name, target, **kwargs)

        @staticmethod
        def _replace_module(parent, child_name, new_module, child):
            if isinstance(child, Autograd4bitQuantLinear) and isinstance(new_module, Linear4bitLt):
                setattr(parent, child_name, new_module)
                _share_quant_tensors(new_module, child)
                _move_adapters(new_module, child.qweight.device)
                return
            return _peft_replace_module(parent, child_name, new_module, child)
else:
    class GPTQLoraModel:
        """Without peft there is no LoraModel to derive from; the two hooks the monkeypatch
        installs are still provided (same signatures as models.py:80-81,116-117) for 4-bit targets."""

        @staticmethod
        def _create_new_module(lora_config, adapter_name, target, **kwargs):
            kwargs.pop("bias", False)
            if not isinstance(target, Autograd4bitQuantLinear):
                raise ValueError(f"Target module {target} is not supported without peft installed.")
            return Linear4bitLt(adapter_name, target.in_features, target.out_features, target.groupsize,
                                target.is_v1_model, **kwargs)

        @staticmethod
        def _replace_module(parent, child_name, new_module, child):
            setattr(parent, child_name, new_module)
            _share_quant_tensors(new_module, child)
            _move_adapters(new_module, child.qweight.device)


def inject_lora_layers(model, target_modules=("q_proj", "v_proj"), r=8, lora_alpha=16, lora_dropout=0.0,
                       adapter_name="default", init_lora_weights=True):
    """peft-free injection: swap every Autograd4bitQuantLinear whose attribute name is in
    `target_modules` for a Linear4bitLt sharing its packed tensors (what get_peft_model does
    through GPTQLoraModel, finetune.py:75-84), freeze everything else, return the new layers."""
    for p in model.parameters():
        p.requires_grad_(False)
    replaced = {}
    for parent_name, parent in list(model.named_modules()):
        for child_name, child in list(parent.named_children()):
            if child_name in target_modules and type(child) is Autograd4bitQuantLinear:
                new = Linear4bitLt(adapter_name, child.in_features, child.out_features, child.groupsize,
                                   child.is_v1_model, r=r, lora_alpha=lora_alpha, lora_dropout=lora_dropout,
                                   init_lora_weights=init_lora_weights)
                GPTQLoraModel._replace_module(parent, child_name, new, child)
                replaced[f"{parent_name}.{child_name}" if parent_name else child_name] = new
    return replaced
