"""Fused q/k/v and gate/up projections: one 4-bit launch instead of three / two, and the whole MLP decode step in one.

Counterpart of make_quant_attn / make_fused_mlp (src/alpaca_lora_4bit/model_attn_mlp_patch.py:73-247 of the
reference), which concatenate the packed tensors of the projections along N and swap in their own attention / MLP
classes.  Two ways here, both leaving the host model's own attention / MLP code in charge:

* in place (the default): the projections stay where they are, on their OWN tensors, and become members of a group.
  At decode sizes (up to 16 rows, no grad) the first member called runs ONE grouped launch for all of them
  (quant_hip.gemv_grouped -> q4_gemv_grouped_f16) and the others pick their result up.  No second copy of the
  weights, the state dict keeps its keys, and members may be LoRA layers (Linear4bitLt): the grouped launch does the
  base products, each member adds its own adapter.  make_fused_mlp also routes the block's forward, at decode sizes,
  through quant_hip.mlp_decode: gate, up, silu(gate) * up and down in one launch.
* `concatenate=True`: the reference's layout.  One new layer holds the N-concatenated tensors and each projection is
  replaced by a slice view of its output (one wider GEMM at prefill sizes as well); `inject_lora_layers(model,
  lora_path)` (model_attn_mlp_patch.py:283-335) then puts a saved q/v adapter onto the fused qkv layer as ONE
  adapter of rank r_q + r_v whose B matrix is block-structured (zero rows for k_proj).
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
    long as the same tensor object comes back unmodified in the same grad mode (identity, in-place version counter),
    whatever the order in which the host block calls its projections, and dropped as soon as every slice has been
    served or the block returns (forward hook installed by _fuse_children), so nothing stays pinned between forwards."""

    def __init__(self, layer, n_slices):
        self.layer = layer
        self.n_slices = n_slices
        self.hook = None
        self.clear()

    def run(self, x):
        key = (x._version, torch.is_grad_enabled())
        if self._x is not x or self._key != key:
            self._y = self.layer(x)
            self._x, self._key, self._served = x, key, 0
        y = self._y
        self._served += 1
        if self._served >= self.n_slices:
            self.clear()
        return y

    def clear(self, *unused):
        self._x = self._y = None
        self._key = None
        self._served = 0


class _MemberGroup:
    """Projections that share their input (q|k|v, gate|up), each on its own tensors.  `run(member, x)` is called from
    Autograd4bitQuantLinear.forward at decode sizes: the first call for an input runs one grouped launch for all
    members, every member takes its own output tensor exactly once (callers add bias and adapter in place)."""

    def __init__(self, members):
        self.members = list(members)
        self.index = {id(m): i for i, m in enumerate(self.members)}
        self.groupsize = self.members[0].groupsize
        self.usable = None                                   # decided at the first call (needs the tensors on the GPU)
        self._layer_cache = None
        self._gemm_ok = None                                 # sequential groups AND scales below 64 (the tiled kernels' fused form)
        self.hook = None
        self.clear()

    def _check(self):
        from . import quant_hip
        try:
            for m in self.members:
                info = quant_hip._layer_info(m.qweight, m.qzeros, m.scales if m.scales.dtype == torch.float16 else m.scales.half(),
                                             m.g_idx, m.groupsize)
                if info.plan is not None or info.gemv_gidx is not None:
                    return False                             # act-order members keep their own launches
        except Exception:
            return False
        return all(m.scales.dtype == torch.float16 for m in self.members)

    def _layers(self):
        """(qweight, qzeros, scales) of every member, rebuilt when a member's buffers were replaced (a cast, a reload)."""
        cached = self._layer_cache
        if cached is not None and all(m._buffers.get('qweight') is c[0] and m._buffers.get('scales') is c[2]
                                      for m, c in zip(self.members, cached)):
            return cached
        self.usable = self._check()
        self._gemm_ok = None
        self._layer_cache = [(m.qweight, m.qzeros, m.scales) for m in self.members] if self.usable else None
        return self._layer_cache

    def run(self, member, x):
        layers = self._layers()
        if layers is None:
            return None
        i = self.index[id(member)]
        if self._x is not x or self._version != x._version or self._outs[i] is None:
            from . import quant_hip
            # the compiled binding checks shapes, dtypes and devices; sequential groups were established by _check()
            outs = quant_hip.gemv_grouped_prepared(x, layers, self.groupsize)
            lead = tuple(x.shape[:-1])
            self._outs = [o.view(lead + (o.shape[-1],)) for o in outs]
            self._x, self._version = x, x._version
        y, self._outs[i] = self._outs[i], None
        if all(o is None for o in self._outs):
            self._x = None
        return y

    def _gemm_spec(self, m, x):
        """How member `m` enters a grouped GEMM for input x: (bias | None, lora_A | None, lora_B | None, scaling, drop_p)."""
        from .autograd_4bit import _is_all_zero
        bias = None
        if not m.disable_bias and not _is_all_zero(m.bias):
            bias = m.bias
        name = None
        if type(m) is not Autograd4bitQuantLinear and not getattr(m, 'disable_adapters', False):
            name = m._fusable_adapter(x)                     # the adapter rides in the launch; otherwise the layer adds it
        if name is None:
            return (bias, None, None, None, 0.0)
        return (bias, m.lora_A[name].weight, m.lora_B[name].weight, float(m.scaling[name]), m._dropout_p(name))

    def run_gemm(self, member, x):
        """Above the decode sizes: ONE grouped GEMM launch for all members (under autograd one node, whose backward is
        one grouped grad-input launch).  Returns the member's output, bias and fused adapter included, or None when
        the group does not take this call (the member then runs by itself)."""
        i = self.index[id(member)]
        key = (x._version, torch.is_grad_enabled())
        if self._gx is x and self._gkey == key and self._gouts[i] is not None:
            y, self._gouts[i] = self._gouts[i], None
            if all(o is None for o in self._gouts):
                self._gx = None
            return y
        from . import autograd_4bit, quant_hip
        layers = self._layers()
        if layers is None or not x.is_cuda or x.shape[-1] != member.in_features:
            return None
        rows = x.numel() // member.in_features
        if rows <= quant_hip.MAX_GEMV_ROWS or not (x.dtype == torch.float16 or torch.is_autocast_enabled('cuda')):
            return None
        if matmul_utils_4bit.use_dense_route(rows) or member.in_features % 128 or any(m.out_features % 128 for m in self.members):
            return None
        Ns = [m.out_features for m in self.members]
        grad = torch.is_grad_enabled()
        if not quant_hip.gemm_grouped_applicable(True, rows, member.in_features, Ns) or \
                (grad and not quant_hip.gemm_grouped_applicable(False, rows, member.in_features, Ns)):
            return None
        if self._gemm_ok is None:
            self._gemm_ok = all(quant_hip._group_layer_ok(l, self.groupsize) for l in layers)
        if not self._gemm_ok:
            return None
        specs, tensors = [], []
        for m, (qweight, qzeros, scales) in zip(self.members, layers):
            bias, la, lb, scaling, drop_p = self._gemm_spec(m, x)
            seed = int(torch.randint(0, 2 ** 62, (1,)).item()) if drop_p > 0.0 else 0
            specs.append((scaling, drop_p, seed))
            tensors += [qweight, scales, qzeros, bias, la, lb]
        outs = autograd_4bit.AutogradMatmul4bitGroup.apply(x, self.groupsize, tuple(specs), *tensors)
        self._gouts = list(outs)
        self._gx, self._gkey = x, key
        y, self._gouts[i] = self._gouts[i], None
        return y

    def clear(self, *unused):
        self._x = None
        self._version = -1
        self._outs = [None] * len(self.members)
        self._gx = None
        self._gkey = None
        self._gouts = [None] * len(self.members)

    def replace(self, old, new):
        """`new` (for instance a LoRA layer sharing `old`'s packed tensors) takes `old`'s place in the group."""
        i = self.index.pop(id(old))
        old.__dict__.pop('_q4_group', None)
        self.members[i] = new
        self.index[id(new)] = i
        new.__dict__['_q4_group'] = self
        self.usable = None
        self._layer_cache = None
        self.clear()


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
    group = _FusedGroup(fused, len(names))
    setattr(parent, fused_name, fused)
    group.hook = parent.register_forward_hook(group.clear)
    start = 0
    for i, (n, m) in enumerate(zip(names, mods)):
        setattr(parent, n, FusedProjectionSlice(group, start, start + m.out_features))
        start += m.out_features
    return True


def _groupable(mods):
    if not all(isinstance(m, Autograd4bitQuantLinear) for m in mods):
        return False                                         # dense projections stay as they are
    first = mods[0]
    return all((m.in_features, m.groupsize, m.bits) == (first.in_features, first.groupsize, first.bits)
               and m.bits == 4 and not m.is_v1_model and m.__dict__.get('_q4_group') is None for m in mods)


def _group_children(parent, names):
    """In-place grouping: the projections keep their tensors and their place; returns the group or None."""
    mods = [getattr(parent, n, None) for n in names]
    if any(m is None for m in mods) or not _groupable(mods):
        return None
    group = _MemberGroup(mods)
    for m in mods:
        m.__dict__['_q4_group'] = group                      # a plain attribute: neither a parameter nor a submodule
    group.hook = parent.register_forward_hook(group.clear)
    return group


def ungroup(model):
    """Undo the in-place grouping (and the MLP decode routing) made by make_quant_attn / make_fused_mlp."""
    count = 0
    for m in model.modules():
        group = m.__dict__.pop('_q4_group', None)
        if group is not None and group.hook is not None:
            group.hook.remove()
            group.hook = None
            count += 1
        if '_q4_mlp_forward' in m.__dict__:
            del m.__dict__['_q4_mlp_forward']
            del m.__dict__['forward']
            m.__dict__.pop('_q4_mlp_args', None)
    return count


def make_quant_attn(model, is_v1_model=False, concatenate=False):
    """One launch for q_proj / k_proj / v_proj of every attention block (model_attn_mlp_patch.py:73-160).
    Returns the number of blocks changed.  In place by default (see the module docstring); `concatenate=True` builds
    the reference's N-concatenated layer and, like the reference (model_attn_mlp_patch.py:78), turns the shared dense
    buffer off -- process-wide: above matmul_utils_4bit.dense_switch_rows rows every product then allocates its own
    dense buffer; set matmul_utils_4bit.cache_buffer = True again if prefill batches of that size matter."""
    if is_v1_model:
        raise NotImplementedError("v1 (fp zeros) layers are not fused")
    names = ("q_proj", "k_proj", "v_proj")
    count = 0
    if concatenate:
        matmul_utils_4bit.cache_buffer = False
    for m in list(model.modules()):
        if all(hasattr(m, n) for n in names):
            count += bool(_fuse_children(m, names, "qkv_proj") if concatenate else _group_children(m, names))
    if concatenate and torch.cuda.is_available():
        torch.cuda.empty_cache()
    return count


# The one-launch MLP step re-reads the intermediate once per output strip of the down projection, which grows with the
# number of rows: measured against grouped gate|up + two elementwise launches + down it wins up to about 4 rows.
mlp_decode_max_rows = 4


def _is_silu(act):
    return isinstance(act, nn.SiLU) or type(act).__name__.lower() in ("silu", "siluactivation") or act is torch.nn.functional.silu


def _plain_no_bias(layer):
    """A 4-bit layer whose forward is the bare product: no active adapter, no bias to add."""
    from .autograd_4bit import _is_all_zero
    if type(layer) is not Autograd4bitQuantLinear:
        if not getattr(layer, 'disable_adapters', False):
            return False
    return layer.disable_bias or _is_all_zero(layer.bias)


def _mlp_decode_args(mlp):
    """(gate, up, down, groupsize, H) for quant_hip's one-launch MLP step, or None when the block does not qualify right
    now: all three layers plain 4-bit products (no active adapter, no bias to add), fp16 scales, sequential groups."""
    from . import quant_hip
    gate, up, down = mlp.gate_proj, mlp.up_proj, mlp.down_proj
    group = gate.__dict__.get('_q4_group')
    if group is None or group._layers() is None:
        return None
    if not all(_plain_no_bias(l) and l.scales.dtype == torch.float16 for l in (gate, up, down)):
        return None
    info = quant_hip._layer_info(down.qweight, down.qzeros, down.scales, down.g_idx, down.groupsize)
    if info.plan is not None or info.gemv_gidx is not None:
        return None
    return ((gate.qweight, gate.qzeros, gate.scales), (up.qweight, up.qzeros, up.scales),
            (down.qweight, down.qzeros, down.scales), int(gate.groupsize), gate.in_features, gate.out_features, down.out_features)


def _mlp_decode_forward(mlp, x):
    """LlamaMLP.forward with the decode step (a few rows, no grad, fp16) as ONE launch: gate, up, silu(gate) * up and
    down (quant_hip.mlp_decode); everything else goes to the block's own forward.  What the step needs of the three
    layers is looked up once and kept while their buffers, adapters and bias switches stay the same objects / values."""
    from . import autograd_4bit, quant_hip
    d = mlp.__dict__
    if (not torch.is_grad_enabled() and x.dtype == torch.float16 and x.is_cuda and autograd_4bit.backend == 'cuda'
            and matmul_utils_4bit.use_new and matmul_utils_4bit.auto_switch):
        cached = d.get('_q4_mlp_args')
        mods = mlp._modules
        gate, up, down = mods['gate_proj'], mods['up_proj'], mods['down_proj']
        bias = [l._buffers.get('bias') for l in (gate, up, down)]
        key = (gate._buffers.get('qweight'), up._buffers.get('qweight'), down._buffers.get('qweight'),
               gate._buffers.get('scales'), bias[0], bias[1], bias[2],
               tuple(-1 if b is None else b._version for b in bias), gate.disable_bias, up.disable_bias, down.disable_bias,
               getattr(gate, 'disable_adapters', None), getattr(up, 'disable_adapters', None), getattr(down, 'disable_adapters', None))
        if cached is None or not (all(a is b for a, b in zip(cached[0][:7], key[:7])) and cached[0][7:] == key[7:]):
            cached = d['_q4_mlp_args'] = (key, _mlp_decode_args(mlp))
        args = cached[1]
        if args is not None and x.shape[-1] == args[4]:
            rows = x.numel() // args[4]
            if (1 <= rows <= min(int(matmul_utils_4bit.auto_switch_thd), quant_hip.MAX_GEMV_ROWS, mlp_decode_max_rows)
                    and quant_hip.mlp_decode_applicable(rows, args[4], args[5], args[3])):
                return quant_hip.mlp_decode_prepared(x, args[0], args[1], args[2], args[3], tuple(x.shape[:-1]) + (args[6],))
    return d['_q4_mlp_forward'](x)


def make_fused_mlp(model, is_v1_model=False, concatenate=False, fuse_decode_step=True):
    """One launch for gate_proj / up_proj of every MLP block (model_attn_mlp_patch.py:163-247; the reference's Triton
    fused-MLP kernel is replaced by one launch over both projections followed by the block's own activation).  In place
    by default; then, with `fuse_decode_step` and a SiLU block of three 4-bit layers of the same group size, the block's
    forward runs the whole decode step (gate, up, silu(gate) * up, down) as one launch."""
    if is_v1_model:
        raise NotImplementedError("v1 (fp zeros) layers are not fused")
    names = ("gate_proj", "up_proj")
    count = 0
    for m in list(model.modules()):
        if all(hasattr(m, n) for n in names + ("down_proj",)):
            if concatenate:
                count += bool(_fuse_children(m, names, "gate_up_proj"))
                continue
            group = _group_children(m, names)
            count += group is not None
            down = m.down_proj
            if (group is not None and fuse_decode_step and _is_silu(getattr(m, 'act_fn', None))
                    and isinstance(down, Autograd4bitQuantLinear) and down.bits == 4 and not down.is_v1_model
                    and down.groupsize == m.gate_proj.groupsize and down.in_features == m.gate_proj.out_features
                    and down.out_features == m.gate_proj.in_features and '_q4_mlp_forward' not in m.__dict__):
                import types
                m.__dict__['_q4_mlp_forward'] = m.forward                # the block's own (bound) forward
                m.__dict__['forward'] = types.MethodType(_mlp_decode_forward, m)
    if concatenate and torch.cuda.is_available():
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
    attention projections.  Same call as the reference's (model_attn_mlp_patch.py:283-335: q_proj and v_proj adapters,
    scaling = lora_alpha / r, a second call replaces the adapter of the first); k_proj adapters are accepted as well.
    On a block fused with `concatenate=True` the adapters become one block-structured adapter on `qkv_proj`; on a block
    grouped in place (or not fused at all) every projection named in the file becomes a LoRA layer of its own that
    shares the projection's packed tensors and keeps its place in the group.  Returns the injected layers."""
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

    def lora_layer(base, a, b):
        # lora_alpha = scaling * rank keeps the layer's own scaling (lora_alpha / r) at the saved adapter's value
        rank = a.shape[0]
        layer = Linear4bitLt('default', base.in_features, base.out_features, base.groupsize, False,
                             r=rank, lora_alpha=scaling * rank, lora_dropout=0.0)
        _share_quant_tensors(layer, base)
        layer.disable_bias = base.disable_bias
        layer.lora_A['default'].weight = nn.Parameter(a, requires_grad=False)
        layer.lora_B['default'].weight = nn.Parameter(b, requires_grad=False)
        layer.is_lora_injected = True
        return layer

    modules = dict(model.named_modules())
    injected = []
    for path, parts in per_block.items():
        attn = modules.get(path)
        if attn is None:
            raise ValueError(f'the adapter names {path}, which the model does not have')
        projs = {n: getattr(attn, n, None) for n in ('q_proj', 'k_proj', 'v_proj')}
        present = [n for n in projs if (n, 'A') in parts and (n, 'B') in parts]
        fused = getattr(attn, 'qkv_proj', None)
        if isinstance(fused, Autograd4bitQuantLinear):       # concatenated block: one block-structured adapter
            rank = sum(parts[(n, 'A')].shape[0] for n in present)
            a_cat = torch.cat([parts[(n, 'A')].to(device=device, dtype=dtype) for n in present], dim=0)
            b_blk = torch.zeros(fused.out_features, rank, device=device, dtype=dtype)
            col = 0
            for n in present:
                b = parts[(n, 'B')].to(device=device, dtype=dtype)
                b_blk[projs[n]._start:projs[n]._stop, col:col + b.shape[1]] = b
                col += b.shape[1]
            layer = lora_layer(fused, a_cat, b_blk)
            attn.qkv_proj = layer
            projs['q_proj']._group.layer = layer
            injected.append(layer)
            continue
        for n in present:                                    # projections on their own tensors
            base = projs[n]
            if not isinstance(base, Autograd4bitQuantLinear) or base.is_v1_model:
                raise ValueError(f'{path}.{n} is not a 4-bit (v2) layer')
            layer = lora_layer(base, parts[(n, 'A')].to(device=device, dtype=dtype), parts[(n, 'B')].to(device=device, dtype=dtype))
            group = base.__dict__.get('_q4_group')
            setattr(attn, n, layer)
            if group is not None:
                group.replace(base, layer)
            injected.append(layer)
    print('Lora Injected.')
    return injected
