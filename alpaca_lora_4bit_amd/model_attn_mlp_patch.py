"""Fused q/k/v and gate/up projections: one wider 4-bit launch instead of three / two.

Counterpart of make_quant_attn / make_fused_mlp (src/alpaca_lora_4bit/model_attn_mlp_patch.py:73-247 of the
reference), which concatenate the packed tensors of the projections along N and swap in their own
attention / MLP classes.  Here the concatenation is the same (fuse_quant_linears), but the host modules
keep their own forward: each original projection is replaced by a slice view of the shared fused layer,
so whatever attention / MLP implementation the installed transformers has calls `q_proj(x)`, `k_proj(x)`,
`v_proj(x)` as before and the first of those calls runs the single fused launch for all three.
At M=1 the fused gate+up GEMV of LLaMA-7B reaches about 50 % of HBM peak against 40 % for two launches.

`inject_lora_layers(model, lora_path)` (model_attn_mlp_patch.py:283-335) puts a saved q/v adapter onto the fused
qkv layers: the per-projection adapters become ONE adapter of rank r_q + r_v whose B matrix is block-structured
(zero rows for k_proj), so the fused layer keeps a single launch sequence.
"""
import json
import os
import re

import torch
import torch.nn as nn

from . import matmul_utils_4bit
from .autograd_4bit import Autograd4bitQuantLinear, fuse_quant_linears


class FusedProjectionSlice(nn.Module):
    """Stands where one projection of a fused group stood; returns its columns of the fused output.
    The fused layer itself is registered once, on the parent module; the slices only point to it."""

    def __init__(self, group, start, stop):
        super().__init__()
        object.__setattr__(self, "_group", group)          # not a registered submodule: no duplicate state
        self.in_features = group.layer.in_features
        self.out_features = stop - start
        self._start, self._stop = start, stop

    def forward(self, x):
        y = self._group.run(x)
        return y[..., self._start:self._stop]


class _FusedGroup:
    """Runs the fused layer once per input tensor and hands the result to every slice.  The result is kept for as
    long as the same tensor object comes back unmodified (identity and in-place version counter), whatever the order
    in which the host block calls its projections; a forward hook on the block (installed by _fuse_children) drops
    it when the block returns, so nothing stays pinned between forwards."""

    def __init__(self, layer):
        self.layer = layer
        self._x = None
        self._version = -1
        self._y = None

    def run(self, x):
        if self._x is not x or self._version != x._version:
            self._y = self.layer(x)
            self._x, self._version = x, x._version
        return self._y

    def clear(self, *unused):
        self._x = self._y = None
        self._version = -1


def _fusable(mods):
    if not all(type(m) is Autograd4bitQuantLinear for m in mods):
        return False                                         # LoRA-wrapped or dense projections stay as they are
    first = mods[0]
    return all((m.in_features, m.groupsize, m.bits) == (first.in_features, first.groupsize, first.bits)
               and not m.is_v1_model and torch.equal(m.g_idx, first.g_idx) for m in mods)


def _fuse_children(parent, names, fused_name):
    mods = [getattr(parent, n, None) for n in names]
    if any(m is None for m in mods) or not _fusable(mods):
        return False
    fused = fuse_quant_linears(mods)
    group = _FusedGroup(fused)
    setattr(parent, fused_name, fused)
    parent.register_forward_hook(group.clear)
    start = 0
    for i, (n, m) in enumerate(zip(names, mods)):
        setattr(parent, n, FusedProjectionSlice(group, start, start + m.out_features))
        start += m.out_features
    return True


def make_quant_attn(model, is_v1_model=False):
    """Fuse q_proj / k_proj / v_proj of every attention block (model_attn_mlp_patch.py:73-160).
    Returns the number of blocks fused.  Like the reference (model_attn_mlp_patch.py:78) it turns the shared dense
    buffer off -- process-wide: above matmul_utils_4bit.dense_switch_rows rows every product then allocates its own
    dense buffer; set matmul_utils_4bit.cache_buffer = True again if prefill batches of that size matter."""
    if is_v1_model:
        raise NotImplementedError("v1 (fp zeros) layers are not fused")
    matmul_utils_4bit.cache_buffer = False
    count = 0
    for m in list(model.modules()):
        if all(hasattr(m, n) for n in ("q_proj", "k_proj", "v_proj")):
            count += _fuse_children(m, ("q_proj", "k_proj", "v_proj"), "qkv_proj")
    if torch.cuda.is_available():
        torch.cuda.empty_cache()
    return count


def make_fused_mlp(model, is_v1_model=False):
    """Fuse gate_proj / up_proj of every MLP block (model_attn_mlp_patch.py:163-247; the reference's Triton
    fused-MLP kernel is replaced by one N-concatenated launch followed by the block's own activation)."""
    if is_v1_model:
        raise NotImplementedError("v1 (fp zeros) layers are not fused")
    count = 0
    for m in list(model.modules()):
        if all(hasattr(m, n) for n in ("gate_proj", "up_proj", "down_proj")):
            count += _fuse_children(m, ("gate_proj", "up_proj"), "gate_up_proj")
    if torch.cuda.is_available():
        torch.cuda.empty_cache()
    return count


def _read_adapter_state(lora_path):
    """Tensors of a saved adapter; only loaders that execute nothing from the file."""
    st = os.path.join(lora_path, "adapter_model.safetensors")
    if os.path.exists(st):
        from safetensors.torch import load_file
        return load_file(st)
    return torch.load(os.path.join(lora_path, "adapter_model.bin"), map_location="cpu", weights_only=True)


_ADAPTER_KEY = re.compile(r"^(?:base_model\.model\.)?(.*)\.(q_proj|k_proj|v_proj)\.lora_([AB])(?:\.[^.]+)?\.weight$")


def inject_lora_layers(model, lora_path, device='cuda', dtype=torch.float16):
    """Loads the adapter saved under `lora_path` (adapter_config.json + adapter_model.safetensors / .bin) onto the
    fused `qkv_proj` layers made by make_quant_attn.  Same call as the reference's
    (model_attn_mlp_patch.py:283-335: q_proj and v_proj adapters, scaling = lora_alpha / r, a second call replaces
    the adapter of the first); k_proj adapters are accepted as well.  Returns the injected layers."""
    from .models import Linear4bitLt, _share_quant_tensors
    print('Device: {}, dtype: {}'.format(device, dtype))
    with open(os.path.join(lora_path, 'adapter_config.json'), 'r') as fh:
        cfg = json.load(fh)
    scaling = cfg['lora_alpha'] / cfg['r']

    per_block = {}                                           # attention module path -> {(proj, 'A'|'B'): tensor}
    for key, tensor in _read_adapter_state(lora_path).items():
        m = _ADAPTER_KEY.match(key)
        if m is not None:
            per_block.setdefault(m.group(1), {})[(m.group(2), m.group(3))] = tensor

    modules = dict(model.named_modules())
    injected = []
    for path, parts in per_block.items():
        attn = modules.get(path)
        fused = getattr(attn, 'qkv_proj', None)
        if not isinstance(fused, Autograd4bitQuantLinear):
            raise ValueError(f'{path} has no fused qkv_proj: call make_quant_attn(model) first')
        slices = {n: getattr(attn, n) for n in ('q_proj', 'k_proj', 'v_proj')}
        present = [n for n in slices if (n, 'A') in parts and (n, 'B') in parts]
        rank = sum(parts[(n, 'A')].shape[0] for n in present)
        a_cat = torch.cat([parts[(n, 'A')].to(device=device, dtype=dtype) for n in present], dim=0)
        b_blk = torch.zeros(fused.out_features, rank, device=device, dtype=dtype)
        col = 0
        for n in present:
            b = parts[(n, 'B')].to(device=device, dtype=dtype)
            b_blk[slices[n]._start:slices[n]._stop, col:col + b.shape[1]] = b
            col += b.shape[1]
        # lora_alpha = scaling * rank keeps the layer's own scaling (lora_alpha / r) at the saved adapter's value
        layer = Linear4bitLt('default', fused.in_features, fused.out_features, fused.groupsize, False,
                             r=rank, lora_alpha=scaling * rank, lora_dropout=0.0)
        _share_quant_tensors(layer, fused)
        layer.disable_bias = fused.disable_bias
        layer.lora_A['default'].weight = nn.Parameter(a_cat, requires_grad=False)
        layer.lora_B['default'].weight = nn.Parameter(b_blk, requires_grad=False)
        layer.is_lora_injected = True
        attn.qkv_proj = layer
        slices['q_proj']._group.layer = layer
        injected.append(layer)
    print('Lora Injected.')
    return injected
