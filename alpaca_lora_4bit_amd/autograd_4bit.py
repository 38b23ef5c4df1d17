"""Quant-linear module and autograd Functions with the interface of the reference's
src/alpaca_lora_4bit/autograd_4bit.py:13-244, running on the gfx950 kernels.

Kept exactly: class names (callers match on `str(type(m))`, finetune.py:101), the 7-argument
`AutogradMatmul4bit.apply(x, qweight, scales, zeros, g_idx, bits, maxq)` with a 7-tuple
backward, the rebindable module globals `AutogradMatmul4bit` / `backend`, buffer names, shapes
and dtypes of `Autograd4bitQuantLinear` (they are the checkpoint format), `switch_backend_to`,
`matmul4bit_with_backend`, `make_quant_for_4bit_autograd`, `model_to_half/float`, `find_layers`.

There is ONE backend and it answers to the name 'cuda' (the torch device string on ROCm, and
what finetune.py:37-40 asks for).  'triton' raises ValueError like an absent Triton does in
the reference (autograd_4bit.py:144-145).
"""
import logging
import math

import torch
import torch.nn as nn
from torch.amp import custom_bwd, custom_fwd

gptq_backend_loaded = False
triton_backend_loaded = False


class AutogradMatmul4bitNotImplemented(torch.autograd.Function):
    """Placeholder bound when the HIP library is missing (autograd_4bit.py:17-26)."""

    @staticmethod
    @custom_fwd(device_type='cuda', cast_inputs=torch.float16)
    def forward(ctx, x, qweight, scales, zeros, g_idx, bits, maxq):
        raise NotImplementedError()

    @staticmethod
    @custom_bwd(device_type='cuda')
    def backward(ctx, grad_output):
        raise NotImplementedError()


try:
    from . import matmul_utils_4bit as mm4b
    from . import quant_hip

    class AutogradMatmul4bitCuda(torch.autograd.Function):
        """y = x @ W with W packed; backward returns dy @ W^T and None for the frozen tensors
        (autograd_4bit.py:32-54).  Only the packed tensors are saved, never a dense W."""

        @staticmethod
        @custom_fwd(device_type='cuda', cast_inputs=torch.float16)
        def forward(ctx, x, qweight, scales, zeros, g_idx, bits, maxq):
            ctx.is_v1 = zeros.dtype != torch.int32
            if ctx.is_v1:                                   # per-column fp zeros: dense dequant + library GEMM
                ctx.save_for_backward(qweight, scales, zeros)
                return mm4b._matmul4bit_v1_recons(x, qweight, scales, zeros)
            ctx.save_for_backward(qweight, scales, zeros, g_idx)
            rows = x.numel() // x.shape[-1]
            if 1 <= rows <= quant_hip.MAX_GEMV_ROWS:
                return mm4b._matmul4bit_v2(x, qweight, scales, zeros, g_idx)
            return mm4b._matmul4bit_v2_recons(x, qweight, scales, zeros, g_idx)

        @staticmethod
        @custom_bwd(device_type='cuda')
        def backward(ctx, grad_output):
            grad = None
            if ctx.is_v1:
                qweight, scales, zeros = ctx.saved_tensors
                if ctx.needs_input_grad[0]:
                    grad = mm4b._matmul4bit_v1_recons(grad_output, qweight, scales, zeros, transpose=True)
                return grad, None, None, None, None, None, None
            qweight, scales, zeros, g_idx = ctx.saved_tensors
            if ctx.needs_input_grad[0]:
                grad = mm4b._matmul4bit_v2_recons(grad_output, qweight, scales, zeros, g_idx, transpose=True)
            return grad, None, None, None, None, None, None

    class AutogradMatmul2bitCuda(torch.autograd.Function):
        """2-bit v2 layers: dense dequant on the GPU + library GEMM, forward and backward
        (autograd_4bit.py:56-72)."""

        @staticmethod
        @custom_fwd(device_type='cuda', cast_inputs=torch.float16)
        def forward(ctx, x, qweight, scales, zeros, g_idx, bits, maxq):
            ctx.save_for_backward(qweight, scales, zeros, g_idx)
            return mm4b._matmul2bit_v2_recons(x, qweight, scales, zeros, g_idx)

        @staticmethod
        @custom_bwd(device_type='cuda')
        def backward(ctx, grad_output):
            qweight, scales, zeros, g_idx = ctx.saved_tensors
            grad = None
            if ctx.needs_input_grad[0]:
                grad = mm4b._matmul2bit_v2_recons(grad_output, qweight, scales, zeros, g_idx, transpose=True)
            return grad, None, None, None, None, None, None

    gptq_backend_loaded = True
except ImportError:
    print('libq4gptq.so not found. Build it with __graft_entry__.build() (hipcc, gfx950).')


def is_triton_backend_available():
    return False


def is_gptq_backend_available():
    return 'AutogradMatmul4bitCuda' in globals()


AutogradMatmul4bit = AutogradMatmul4bitNotImplemented
AutogradMatmul2bit = AutogradMatmul4bitNotImplemented
backend = None
if is_gptq_backend_available():
    AutogradMatmul4bit = AutogradMatmul4bitCuda
    AutogradMatmul2bit = AutogradMatmul2bitCuda
    backend = 'cuda'
else:
    logging.warning("The gfx950 4-bit backend is not available.")


def switch_backend_to(to_backend):
    global AutogradMatmul4bit
    global backend
    if to_backend == 'cuda':
        if not is_gptq_backend_available():
            raise ValueError('libq4gptq.so not found. Build it with __graft_entry__.build().')
        AutogradMatmul4bit = AutogradMatmul4bitCuda
        backend = 'cuda'
        print('Using the gfx950 HIP implementation (backend name: cuda).')
    elif to_backend == 'triton':
        raise ValueError('Triton not found. This build has a single HIP backend; use "cuda".')
    else:
        raise ValueError('Backend not supported.')


def matmul4bit_with_backend(x, qweight, scales, qzeros, g_idx, bits, maxq, groupsize=None):
    if backend == 'cuda':
        return mm4b.matmul4bit(x, qweight, scales, qzeros, g_idx, groupsize)
    raise ValueError('Backend not supported.')


def _is_all_zero(bias):
    """True when `bias` holds only zeros, which is what checkpoints without biases leave in the buffer
    (autograd_4bit.py:186): the in-place add of the reference's forward (:207-208) is then skipped.  The verdict
    is kept on the tensor object with its in-place version counter; the first call per tensor synchronises."""
    key = (bias._version, bias.data_ptr())
    cached = getattr(bias, "_q4_zero", None)
    if cached is not None and cached[0] == key:
        return cached[1]
    if torch.cuda.is_available() and bias.is_cuda and torch.cuda.is_current_stream_capturing():
        return False                  # no synchronising reduction inside a graph capture: keep the add
    verdict = not bool(bias.any())
    try:
        bias._q4_zero = (key, verdict)
    except AttributeError:
        pass
    return verdict


class Autograd4bitQuantLinear(nn.Module):
    """GPTQ 4-bit linear layer; buffers as registered at autograd_4bit.py:166-189."""

    def __init__(self, in_features, out_features, groupsize=-1, is_v1_model=False, bits=4):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.bits = bits
        self.maxq = 2 ** self.bits - 1
        groupsize = groupsize if groupsize != -1 else in_features
        self.groupsize = groupsize
        self.is_v1_model = is_v1_model
        self.disable_bias = False
        n_groups = math.ceil(in_features / groupsize)
        if is_v1_model:
            self.register_buffer('zeros', torch.empty((out_features, 1)))
            self.register_buffer('scales', torch.empty((out_features, 1)))
            self.g_idx = None
        else:
            self.register_buffer('qzeros', torch.empty((n_groups, out_features * bits // 32), dtype=torch.int32))
            self.register_buffer('scales', torch.empty((n_groups, out_features)))
            self.register_buffer('g_idx', (torch.arange(in_features, dtype=torch.int64) // groupsize).to(torch.int32))
        self.register_buffer('bias', torch.zeros(out_features))
        self.register_buffer('qweight', torch.empty((in_features * bits // 32, out_features), dtype=torch.int32))

    def forward(self, x):
        if (self.bits == 4 and not self.is_v1_model and x.dtype == torch.float16 and backend == 'cuda'
                and not torch.is_grad_enabled() and mm4b.use_new and mm4b.auto_switch):
            # decode: the same call matmul4bit -> _matmul4bit_v2 would end in, without the stops on the way
            rows = x.numel() // self.in_features if self.in_features else 0
            if 1 <= rows <= min(int(mm4b.auto_switch_thd), quant_hip.MAX_GEMV_ROWS) and x.shape[-1] == self.in_features:
                scales = self.scales
                # a member of a group made by model_attn_mlp_patch (q|k|v, gate|up): the first member called runs ONE
                # launch over every member's own tensors and the others pick their result up
                group = self.__dict__.get('_q4_group')
                out = group.run(self, x) if group is not None else None
                if out is None:
                    out = quant_hip.gemv(x, self.qweight, self.qzeros, scales if scales.dtype == torch.float16 else scales.half(),
                                         self.g_idx, self.groupsize, out_shape=x.shape[:-1] + (self.out_features,))
                if not self.disable_bias and not _is_all_zero(self.bias):
                    out += self.bias
                return out
        group = self.__dict__.get('_q4_group')
        if group is not None and self.bits == 4 and not self.is_v1_model and backend == 'cuda':
            # a member of a group made by model_attn_mlp_patch, above the decode sizes: one grouped GEMM launch for
            # all members (forward and, under autograd, grad-input), each member picks its output up
            out = group.run_gemm(self, x)
            if out is not None:
                return out
        zeros = self.zeros if self.is_v1_model else self.qzeros
        if self.bits == 4:
            if torch.is_grad_enabled():
                out = AutogradMatmul4bit.apply(x, self.qweight, self.scales, zeros, self.g_idx, self.bits, self.maxq)
            else:
                out = matmul4bit_with_backend(x, self.qweight, self.scales, zeros, self.g_idx, self.bits, self.maxq,
                                              self.groupsize)
        elif self.bits == 2:
            out = AutogradMatmul2bit.apply(x, self.qweight, self.scales, self.qzeros, self.g_idx, self.bits, self.maxq)
        else:
            raise ValueError('Unsupported bitwidth.')
        if not self.disable_bias and not _is_all_zero(self.bias):
            out += self.bias
        return out


def make_quant_for_4bit_autograd(module, names, name='', groupsize=-1, is_v1_model=False, bits=4):
    """Replace every attribute of `module` (recursively) whose dotted path is in `names` by an
    empty Autograd4bitQuantLinear of the same in/out features (autograd_4bit.py:211-222)."""
    if isinstance(module, Autograd4bitQuantLinear):
        return
    for child_name, child in list(module.named_children()):
        path = f'{name}.{child_name}' if name else child_name
        if path in names:
            setattr(module, child_name, Autograd4bitQuantLinear(child.in_features, child.out_features,
                                                                groupsize=groupsize, is_v1_model=is_v1_model, bits=bits))
        else:
            make_quant_for_4bit_autograd(child, names, path, groupsize=groupsize, is_v1_model=is_v1_model, bits=bits)


def fuse_quant_linears(layers):
    """One Autograd4bitQuantLinear computing the concatenation of the outputs of `layers`
    (same in_features, groupsize and g_idx): q/k/v or gate/up as a single, wider launch.
    Every packed tensor is N-minor, so the fusion is a plain concatenation along N; it is what the
    reference's make_quant_attn / make_fused_mlp do (model_attn_mlp_patch.py:88-100, 180-190)."""
    first = layers[0]
    for l in layers[1:]:
        if (l.in_features, l.groupsize, l.bits, l.is_v1_model) != (first.in_features, first.groupsize, first.bits,
                                                                   first.is_v1_model):
            raise ValueError('layers to fuse must share in_features, groupsize, bits and layout')
        if first.is_v1_model or not torch.equal(l.g_idx, first.g_idx):
            raise ValueError('layers to fuse must be v2 layers with identical g_idx')
    fused = Autograd4bitQuantLinear(first.in_features, sum(l.out_features for l in layers), groupsize=first.groupsize,
                                    is_v1_model=False, bits=first.bits)
    fused.qweight = torch.cat([l.qweight for l in layers], dim=1).contiguous()
    fused.qzeros = torch.cat([l.qzeros for l in layers], dim=1).contiguous()
    fused.scales = torch.cat([l.scales for l in layers], dim=1).contiguous()
    fused.bias = torch.cat([l.bias for l in layers], dim=0).contiguous()
    fused.g_idx = first.g_idx
    fused.disable_bias = all(l.disable_bias for l in layers)
    return fused


def _cast_quant_buffers(model, dtype):
    for _, m in model.named_modules():
        if isinstance(m, Autograd4bitQuantLinear):
            if gptq_backend_loaded:
                quant_hip.invalidate(m)                    # whatever was cached about the old buffers goes with them
            if m.is_v1_model:
                m.zeros = m.zeros.to(dtype)
            m.scales = m.scales.to(dtype)
            m.bias = m.bias.to(dtype)


def model_to_half(model):
    """autograd_4bit.py:225-233."""
    model.half()
    _cast_quant_buffers(model, torch.float16)
    print('Converted as Half.')


def model_to_float(model):
    """autograd_4bit.py:236-244.  Note: the HIP kernels take fp16 scales; fp32 scales are
    rounded to fp16 on every call, so prefer model_to_half."""
    model.float()
    _cast_quant_buffers(model, torch.float32)
    print('Converted as Float.')


def find_layers(module, layers=(nn.Conv2d, nn.Linear), name=''):
    """{dotted name: module} of every leaf whose exact type is in `layers` (autograd_4bit.py:247-255)."""
    if type(module) in layers:
        return {name: module}
    res = {}
    for child_name, child in module.named_children():
        res.update(find_layers(child, layers=layers, name=f'{name}.{child_name}' if name else child_name))
    return res


class AutogradMatmul4bitLora(torch.autograd.Function):
    """Fused  y = x @ W (+ bias) + scaling * (x @ A^T) @ B^T  for one LoRA adapter.

    No counterpart in the reference as a single op: it is Autograd4bitQuantLinear.forward
    (autograd_4bit.py:192-208) followed by the adapter lines of Linear4bitLt.forward
    (models.py:58-66) and, in backward, AutogradMatmul4bitCuda.backward (autograd_4bit.py:45-54)
    plus torch autograd over the two adapter Linears.  Here the rank-r products ride in the
    main GEMM as one extra reduction step, forward and backward:
        fwd   xa  = x @ A^T    [M, r]   then  y  = [x | xa]  @ [W ; scaling * B^T]
        bwd   dyb = dy @ B     [M, r]   then  dx = [dy | dyb] @ [W^T ; scaling * A]
              dA  = scaling * dyb^T @ x   [r, K]        dB = scaling * dy^T @ xa   [N, r]
    A: lora_A.weight [r, K], B: lora_B.weight [N, r] (any float dtype; products run in fp16
    with fp32 accumulation, like the reference under autocast).  fp32 / fp16 adapter matrices are
    read in place by the kernels through strides: no cast, transposed or pre-scaled copies.

    With matmul_utils_4bit.dense_switch_rows set, above that many rows the same sums run as dense dequantization + library GEMMs
    (the rank-r product writes the output once, the big product accumulates onto it).

    Dropout in front of lora_A (models.py:63-66; the reference's default is p = 0.05, arg_parser.py:48) stays
    inside the same kernels: with drop_p > 0 the adapter sees xd = dropout(x) under a mask that is a pure
    function of (drop_seed, row, column) and is regenerated wherever it is needed instead of being stored:
        fwd   xa = xd @ A^T                       bwd   dA = scaling * dyb^T @ xd
              dx = dy @ W^T + mask/(1-p) * (scaling * dyb @ A)          dB = scaling * dy^T @ xa"""

    @staticmethod
    def _kernel_dtype(w):
        return w if w.dtype in (torch.float16, torch.float32) else w.float()

    @staticmethod
    def _dense_product(act, w, small, adapter, scaling, bias=None):
        """act @ w + scaling * small @ adapter (+ bias), fp16 out; `w`, `adapter` may be transposed views."""
        adapter = adapter if adapter.dtype == torch.float16 else adapter.to(torch.float16)
        if bias is not None:
            out = torch.addmm(bias, small, adapter, alpha=scaling)
        else:
            out = torch.mm(small * scaling, adapter)
        return out.addmm_(act, w)

    @staticmethod
    def _adapter_grads(dyb, x2, xa, dy, scaling, dropout, need_a, need_b, ab_dtypes):
        """(dA, dB) = scaling * (dyb^T @ dropout(x), dy^T @ xa) in the parameters' dtypes (None where not needed)."""
        da = db = None
        r = dyb.shape[1]
        if need_a and need_b and r in quant_hip.LORA_GRAD_RANKS:
            da, db = quant_hip.lora_grad_pair(dyb, x2, xa, dy, scaling, dropout=dropout)   # one launch for both gradients
        else:
            if need_a:
                if r in quant_hip.LORA_GRAD_RANKS:
                    da = quant_hip.lora_grad(dyb, x2, scaling, dropout=dropout)
                elif dropout is not None:
                    xd = x2 * quant_hip.dropout_keep_mask(x2.shape[0], x2.shape[1], dropout[0], dropout[1], x2.device)
                    da = torch.mm(dyb.t(), xd).float().mul_(scaling * quant_hip.dropout_scale(dropout[1]))
                else:
                    da = torch.mm(dyb.t(), x2).float().mul_(scaling)
            if need_b:
                if r in quant_hip.LORA_GRAD_RANKS:
                    db = quant_hip.lora_grad(xa, dy, scaling, transposed=True)
                else:
                    db = torch.mm(dy.t(), xa).float().mul_(scaling)
        if da is not None:
            da = da.to(ab_dtypes[0])
        if db is not None:
            db = db.to(ab_dtypes[1])
        return da, db

    @staticmethod
    @custom_fwd(device_type='cuda', cast_inputs=None)
    def forward(ctx, x, qweight, scales, zeros, g_idx, bias, lora_a, lora_b, scaling, groupsize, drop_p=0.0,
                drop_seed=0):
        K, N = qweight.shape[0] * 8, qweight.shape[1]
        dropout = (int(drop_seed), float(drop_p)) if drop_p and drop_p > 0.0 else None
        x2 = x.reshape(-1, K)
        if x2.dtype != torch.float16:
            x2 = x2.half()
        x2 = x2.contiguous()
        if bias is not None and bias.dtype != torch.float16:
            bias = bias.half()
        a = AutogradMatmul4bitLora._kernel_dtype(lora_a.detach())
        b = AutogradMatmul4bitLora._kernel_dtype(lora_b.detach())
        xa = quant_hip.lora_down(x2, a, dropout=dropout)
        if mm4b.use_dense_route(x2.shape[0]):
            w = mm4b.dense_weight(qweight, scales, zeros, g_idx, groupsize)
            y = AutogradMatmul4bitLora._dense_product(x2, w, xa, b.t(), scaling, bias).view(tuple(x.shape[:-1]) + (N,))
        else:
            y = quant_hip.gemm_fwd(x2, qweight, zeros, scales, g_idx, groupsize, bias=bias,
                                   xa=xa, lora_bt=b.t(), lora_scale=scaling, out_shape=tuple(x.shape[:-1]) + (N,))
        ctx.save_for_backward(x2, xa, qweight, scales, zeros, g_idx, a, b)
        ctx.scaling = scaling
        ctx.groupsize = groupsize
        ctx.ab_dtypes = (lora_a.dtype, lora_b.dtype)
        ctx.dropout = dropout
        return y

    @staticmethod
    @custom_bwd(device_type='cuda')
    def backward(ctx, grad_output):
        x2, xa, qweight, scales, zeros, g_idx, a, b = ctx.saved_tensors
        N = qweight.shape[1]
        dy = grad_output.reshape(-1, N)
        if dy.dtype != torch.float16:
            dy = dy.half()
        dy = dy.contiguous()
        dyb = quant_hip.lora_down(dy, b.t())
        dropout = ctx.dropout
        dx = da = db = None
        r = a.shape[0]
        need_a, need_b = ctx.needs_input_grad[6], ctx.needs_input_grad[7]
        if ctx.needs_input_grad[0]:
            dx_shape = tuple(grad_output.shape[:-1]) + (qweight.shape[0] * 8,)
            if mm4b.use_dense_route(dy.shape[0]):
                w = mm4b.dense_weight(qweight, scales, zeros, g_idx, ctx.groupsize)
                if dropout is None:
                    dx = AutogradMatmul4bitLora._dense_product(dy, w.t(), dyb, a, ctx.scaling).view(dx_shape)
                else:
                    dx = quant_hip.masked_adapter_term(dyb, a, ctx.scaling, dropout).addmm_(dy, w.t()).view(dx_shape)
            else:
                dx = quant_hip.gemm_bwd_dx(dy, qweight, zeros, scales, g_idx, ctx.groupsize, dyb=dyb, lora_a=a,
                                           lora_scale=ctx.scaling, out_shape=dx_shape, dropout=dropout)
        da, db = AutogradMatmul4bitLora._adapter_grads(dyb, x2, xa, dy, ctx.scaling, dropout, need_a, need_b, ctx.ab_dtypes)
        return dx, None, None, None, None, None, da, db, None, None, None, None


class AutogradMatmul4bitGroup(torch.autograd.Function):
    """The products of 2..4 layers that share their input (q|k|v, gate|up of a decoder block), LoRA adapters included,
    as ONE node: forward = one grouped launch on the layers' own tensors, backward = one grouped grad-input launch
    whose ordered reduction also does the sum over the layers that autograd would otherwise add up.

    No counterpart in the reference as a single op; per layer it computes what AutogradMatmul4bitCuda
    (autograd_4bit.py:32-54) and, for a layer with an adapter, the adapter lines of Linear4bitLt.forward
    (models.py:58-66) compute, and the reference reaches the single launch by concatenating the packed tensors
    (model_attn_mlp_patch.py:88-100, 180-190).

    apply(x, groupsize, specs, *tensors): specs[i] = (scaling | None, drop_p, drop_seed) of layer i; tensors holds six
    entries per layer: qweight, scales, qzeros, bias | None, lora_A.weight | None, lora_B.weight | None.
    Returns one output per layer."""

    @staticmethod
    @custom_fwd(device_type='cuda', cast_inputs=None)
    def forward(ctx, x, groupsize, specs, *tensors):
        n = len(specs)
        lay = [tensors[6 * i:6 * i + 6] for i in range(n)]
        K = lay[0][0].shape[0] * 8
        x2 = x.reshape(-1, K)
        if x2.dtype != torch.float16:
            x2 = x2.half()
        x2 = x2.contiguous()
        fwd, xas, adapters, dropouts = [], [], [], []
        for (qweight, scales, zeros, bias, lora_a, lora_b), (scaling, drop_p, drop_seed) in zip(lay, specs):
            if bias is not None and bias.dtype != torch.float16:
                bias = bias.half()
            dropout = (int(drop_seed), float(drop_p)) if drop_p and drop_p > 0.0 else None
            if lora_a is not None:
                a = AutogradMatmul4bitLora._kernel_dtype(lora_a.detach())
                b = AutogradMatmul4bitLora._kernel_dtype(lora_b.detach())
                xa = quant_hip.lora_down(x2, a, dropout=dropout)
                fwd.append((qweight, zeros, scales, bias, xa, b.t(), scaling))
            else:
                a = b = xa = None
                fwd.append((qweight, zeros, scales, bias, None, None, 1.0))
            xas.append(xa); adapters.append((a, b)); dropouts.append(dropout)
        ys = quant_hip.gemm_grouped_fwd(x2, fwd, groupsize)
        lead = tuple(x.shape[:-1])
        saved = [x2]
        for (qweight, scales, zeros, _, _, _), xa, (a, b) in zip(lay, xas, adapters):
            saved += [qweight, scales, zeros] + ([xa, a, b] if a is not None else [])
        ctx.save_for_backward(*saved)
        ctx.specs = specs
        ctx.groupsize = groupsize
        ctx.has_adapter = [a is not None for a, _ in adapters]
        ctx.dropouts = dropouts
        ctx.ab_dtypes = [(l[4].dtype, l[5].dtype) if l[4] is not None else None for l in lay]
        return tuple(y.view(lead + (y.shape[-1],)) for y in ys)

    @staticmethod
    @custom_bwd(device_type='cuda')
    def backward(ctx, *grad_outputs):
        saved = list(ctx.saved_tensors)
        x2 = saved.pop(0)
        n = len(ctx.specs)
        grads = [None] * (6 * n)
        layers, dys, per_layer = [], [], []
        for i in range(n):
            qweight, scales, zeros = saved.pop(0), saved.pop(0), saved.pop(0)
            xa = a = b = None
            if ctx.has_adapter[i]:
                xa, a, b = saved.pop(0), saved.pop(0), saved.pop(0)
            N = qweight.shape[1]
            g = grad_outputs[i]
            if g is None:
                dy = torch.zeros((x2.shape[0], N), dtype=torch.float16, device=x2.device)
            else:
                dy = g.reshape(-1, N)
                if dy.dtype != torch.float16:
                    dy = dy.half()
                dy = dy.contiguous()
            dyb = quant_hip.lora_down(dy, b.t()) if a is not None else None
            dys.append(dy)
            layers.append((qweight, zeros, scales, dyb, a, ctx.specs[i][0] if a is not None else 1.0, ctx.dropouts[i]))
            per_layer.append((xa, dyb, dy))
        dx = None
        if ctx.needs_input_grad[0]:
            lead = next((tuple(g.shape[:-1]) for g in grad_outputs if g is not None), (x2.shape[0],))
            dx = quant_hip.gemm_grouped_bwd_dx(dys, layers, ctx.groupsize, out_shape=lead + (x2.shape[1],))
        for i in range(n):
            if ctx.has_adapter[i]:
                xa, dyb, dy = per_layer[i]
                need_a, need_b = ctx.needs_input_grad[3 + 6 * i + 4], ctx.needs_input_grad[3 + 6 * i + 5]
                if need_a or need_b:
                    grads[6 * i + 4], grads[6 * i + 5] = AutogradMatmul4bitLora._adapter_grads(
                        dyb, x2, xa, dy, ctx.specs[i][0], ctx.dropouts[i], need_a, need_b, ctx.ab_dtypes[i])
        return (dx, None, None) + tuple(grads)


_LOADER_NAMES = ('load_llama_model_4bit_low_ram', 'load_llama_model_4bit_low_ram_and_offload',
                 'load_llama_model_4bit_low_ram_and_offload_to_cpu')


def __getattr__(name):
    # the reference defines its loaders in this module (autograd_4bit.py:250-360); here they live in
    # loaders.py (which imports this module) and are resolved lazily under the same names
    if name in _LOADER_NAMES:
        from . import loaders
        return getattr(loaders, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
