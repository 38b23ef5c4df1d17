"""Host dispatch for the 4-bit matmul: same functions and module-level knobs as the reference's
src/alpaca_lora_4bit/matmul_utils_4bit.py, routed to the gfx950 kernels.

What changed underneath (none of it visible in the signatures):

* rows <= auto_switch_thd (default 16, the most the GEMV kernel takes) go to one GEMV launch
  that reads the packed weights once for all rows; the reference launches one grid slice per row
  and switches to recons + matmul above 8 rows (matmul_utils_4bit.py:15,164-167).
* larger inputs go to the fused dequant + MFMA GEMM, which needs no dense [K, N] buffer.
* the reference's own scheme (dense dequantization into a buffer from `get_buffer`, then a library GEMM) is kept
  behind `dense_switch_rows`: rows above that value take it.  The default is None (never): with 256 x 256 tiles for
  large outputs the fused kernel is level with dequantization + library GEMM from 2560 rows up (a 7B decoder
  layer's seven products, forward + grad-input: 5 % faster at 4096 rows, 4 % slower at 8192) and needs no dense
  buffer.  Layers whose in / out features are not multiples of 128 always take the dense route.  `cache_buffer`
  keeps its meaning (one process-global buffer per shape, or a fresh one per call when False).
* `act_order` and `faster_mode` no longer select kernels: whether `g_idx` is a real
  permutation is detected per tensor (quant_hip.classify_g_idx).  The reference's default
  kernel ignores g_idx unless the user sets `act_order = True` by hand (:75-87); here a
  permuted g_idx is always honoured.
"""
import logging

import numpy as np
import torch

try:
    from . import quant_hip
except (ImportError, ModuleNotFoundError) as e:   # same convention as matmul_utils_4bit.py:5-9
    logging.exception("libq4gptq.so is not built: run __graft_entry__.build()")
    raise e

# Global knobs (names and defaults of matmul_utils_4bit.py:11-20; see the module docstring)
buffer_mat_dic = {}
use_new = True
auto_switch = True
auto_switch_thd = 16
debug = False
faster_mode = 'old_faster'
valid_faster_mode = ('faster', 'old_faster')
act_order = False
cache_buffer = True
dense_switch_rows = None          # rows above this: dense dequant + library GEMM; 0 or None: always the fused GEMM


def get_buffer(shape_of_qweight, dtype=torch.float16, device='cuda', bits=4, zero=True):
    """Dense [K, N] scratch of the reference (matmul_utils_4bit.py:22-33): used above `dense_switch_rows` rows
    and by callers that dequantize explicitly.  Like the reference's, the cached buffer is shared by every layer
    of that shape, so calls on two streams at once must set `cache_buffer = False`."""
    target_shape = (shape_of_qweight[0] * (32 // bits), shape_of_qweight[1])
    make = torch.zeros if zero else torch.empty
    if not cache_buffer:
        return make(target_shape, dtype=dtype, device=device)
    device = torch.device(device)
    if device.type == 'cuda' and device.index is None:
        device = torch.device('cuda', torch.cuda.current_device())
    key = (target_shape, device)
    buf = buffer_mat_dic.get(key)
    if buf is None or buf.dtype != dtype:
        buf = make(target_shape, dtype=dtype, device=device)
        buffer_mat_dic[key] = buf
    return buf


def _rows(x):
    """Number of rows of x seen as a matrix [rows, K] (np.prod(x.shape[:-1]) of the reference)."""
    return x.numel() // x.shape[-1] if x.shape[-1] else 0


def _groupsize_of(qweight, scales, groupsize):
    if groupsize is not None and groupsize > 0:
        return int(groupsize)
    K, G = qweight.shape[0] * 8, scales.shape[0]
    return -(-K // G)


def _half_scales(scales):
    return scales if scales.dtype == torch.float16 else scales.half()


def _matmul4bit_v2(x, qweight, scales, zeros, g_idx, groupsize=None):
    """x @ W for a handful of rows (decode).  matmul_utils_4bit.py:59-95."""
    if debug:
        print('_matmul4bit_v2')
    assert qweight.shape[0] * 8 == x.shape[-1]
    if faster_mode not in valid_faster_mode and faster_mode != 'disable':
        raise ValueError('faster_mode should be in {}'.format(valid_faster_mode))
    outshape = x.shape[:-1] + (qweight.shape[1],)
    dtype = x.dtype
    y = quant_hip.gemv(x, qweight, zeros, _half_scales(scales), g_idx, _groupsize_of(qweight, scales, groupsize),
                       out_shape=outshape)
    return y.to(dtype)


def use_dense_route(rows):
    """True when `rows` activation rows go through dense dequantization + a library GEMM."""
    return bool(dense_switch_rows) and rows > dense_switch_rows


def dense_weight(qweight, scales, zeros, g_idx, groupsize=None):
    """W fp16 [K, N] in the buffer of `get_buffer` (every element is overwritten)."""
    buf = get_buffer(qweight.shape, dtype=torch.float16, device=qweight.device, zero=False)
    return quant_hip.dequant(qweight, zeros, _half_scales(scales), g_idx, _groupsize_of(qweight, scales, groupsize),
                             out=buf)


def _matmul4bit_v2_recons(x, qweight, scales, zeros, g_idx, transpose=False, groupsize=None):
    """x @ W (or x @ W.T with transpose=True).  Up to `dense_switch_rows` rows through the fused dequant-MFMA GEMM;
    above, as the reference does for every size: dequantize into a dense buffer and call torch.matmul
    (matmul_utils_4bit.py:114-127)."""
    if debug:
        print('_matmul4bit_v2_recons')
    if not transpose:
        assert qweight.shape[0] * 8 == x.shape[-1]
    else:
        assert qweight.shape[1] == x.shape[-1]
    gs = _groupsize_of(qweight, scales, groupsize)
    lead = tuple(x.shape[:-1])
    # layers whose in / out features are not multiples of 128 are outside the tiled kernels: they take the dense route
    # at every size (the dequantization needs only K % 32 == 0 and N % 64 == 0), as the reference does for every layer
    odd_shape = (qweight.shape[0] * 8) % 128 != 0 or qweight.shape[1] % 128 != 0
    if (use_dense_route(_rows(x)) or odd_shape) and x.is_cuda:
        return _dense_matmul(x, dense_weight(qweight, scales, zeros, g_idx, gs), transpose)
    if not transpose:
        return quant_hip.gemm_fwd(x, qweight, zeros, _half_scales(scales), g_idx, gs,
                                  out_shape=lead + (qweight.shape[1],))
    return quant_hip.gemm_bwd_dx(x, qweight, zeros, _half_scales(scales), g_idx, gs,
                                 out_shape=lead + (qweight.shape[0] * 8,))


def _dense_matmul(x, w, transpose):
    # the dense buffer is fp16; activations follow it (the reference multiplies in the buffer's dtype)
    xh = x if x.dtype == torch.float16 else x.half()
    return torch.matmul(xh, w.t() if transpose else w)


def _matmul4bit_v1_recons(x, qweight, scales, zeros, transpose=False):
    """v1 layers (one fp scale / zero per column): dense dequant on the GPU, then a library GEMM
    (matmul_utils_4bit.py:98-111).  The fused kernels of this package cover the v2 layout only."""
    if not transpose:
        assert qweight.shape[0] * 8 == x.shape[-1]
    else:
        assert qweight.shape[1] == x.shape[-1]
    return _dense_matmul(x, quant_hip.dequant_v1(qweight, scales, zeros), transpose)


def _matmul4bit_v1(x, qweight, scales, zeros):
    """x @ W of a v1 layer for a handful of rows (matmul_utils_4bit.py:36-56); more rows than the GEMV takes go
    through the dense path."""
    assert qweight.shape[0] * 8 == x.shape[-1]
    if _rows(x) > quant_hip.MAX_GEMV_ROWS:
        return _matmul4bit_v1_recons(x, qweight, scales, zeros).to(x.dtype)
    outshape = x.shape[:-1] + (qweight.shape[1],)
    return quant_hip.gemv_v1(x, qweight, scales, zeros, out_shape=outshape).to(x.dtype)


def _matmul2bit_v2_recons(x, qweight, scales, zeros, g_idx, transpose=False):
    """2-bit v2 layers: dense dequant + library GEMM (matmul_utils_4bit.py:130-143)."""
    if not transpose:
        assert qweight.shape[0] * 16 == x.shape[-1]
    else:
        assert qweight.shape[1] == x.shape[-1]
    return _dense_matmul(x, quant_hip.dequant2(qweight, zeros, _half_scales(scales), g_idx), transpose)


def v2_to_v1(scales, zeros):
    """Zero points of a single-group v2 layer as v1 fp zeros: scales * (z + 1)
    (matmul_utils_4bit.py:173-186, which builds the same numbers through vecquant4recons_v1)."""
    assert zeros.shape[0] == 1
    N = scales.shape[-1]
    shifts = (torch.arange(N, device=zeros.device) % 8) * 4
    z = (zeros.reshape(-1)[torch.arange(N, device=zeros.device) // 8] >> shifts) & 0xF
    return z.to(torch.float16) * scales + scales


def matmul4bit(x, qweight, scales, zeros, g_idx=None, groupsize=None):
    """No-grad dispatcher, matmul_utils_4bit.py:146-170."""
    if zeros.dtype != torch.int32:
        # v1 layout (matmul_utils_4bit.py:148-156): decode sizes take the GEMV, the rest dense dequant + GEMM
        rows = _rows(x)
        thd = min(int(auto_switch_thd), quant_hip.MAX_GEMV_ROWS) if (use_new and auto_switch) else quant_hip.MAX_GEMV_ROWS
        if 1 <= rows <= thd:
            return _matmul4bit_v1(x, qweight, scales, zeros)
        return _matmul4bit_v1_recons(x.half(), qweight, scales.half(), zeros.half())
    gs = _groupsize_of(qweight, scales, groupsize)
    rows = _rows(x)
    thd = min(int(auto_switch_thd), quant_hip.MAX_GEMV_ROWS)
    use_gemv = rows <= thd if (use_new and auto_switch) else rows <= quant_hip.MAX_GEMV_ROWS
    if use_gemv and rows >= 1:
        return _matmul4bit_v2(x, qweight, scales, zeros, g_idx, gs)
    return _matmul4bit_v2_recons(x.half(), qweight, scales.half(), zeros, g_idx, groupsize=gs)
