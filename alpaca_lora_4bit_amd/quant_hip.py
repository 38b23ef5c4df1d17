"""Tensor-level host side of libq4gptq: the stand-in for the reference's `quant_cuda` module.

Two layers:

* `dequant`, `gemv`, `gemm_fwd`, `gemm_bwd_dx` -- the operators the rest of this package uses.
  They do the checks the reference's C++ binding leaves out (dtype, device, contiguity, shape,
  g_idx range), pick torch's CURRENT stream for the tensor's device, and call the C ABI.
* `vecquant4recons_v2`, `vecquant4matmul`, `vecquant4matmul_faster`, `vecquant4matmul_old_faster`
  -- same names, argument order and "write into the caller's buffer, return None" convention as
  the pybind functions of src/alpaca_lora_4bit/quant_cuda/quant_cuda.cpp:204-227, so code
  written against `quant_cuda` keeps working.

Nothing here computes on the CPU: without the built library the import fails.
"""
from __future__ import annotations

import ctypes

import torch

from . import _lib
from ._lib import Q4Error  # noqa: F401  (re-exported)

_lib.lib()  # fail at import time, loudly, if the HIP library is missing

# Compiled host binding (csrc/host/q4_host.cpp, built by g++ next to the library): does the per-call checks, takes
# torch's current stream, keeps the workspaces and calls the C ABI without going through ctypes.  The ctypes path
# below stays as the fallback for a tree where only the library was built.
try:
    from . import _q4_host as _host
    if _host.abi_version() != _lib.ABI_VERSION:
        raise ImportError(f"_q4_host was built against ABI {_host.abi_version()}, the library has {_lib.ABI_VERSION}; rebuild")
    _host.set_error_class(_lib.Q4Error)
except ModuleNotFoundError:
    _host = None

MAX_GEMV_ROWS = 16
MAX_GEMV_SORTED_ROWS = 3          # q4_gemv_sorted_f16 (x gathered inside the kernel) wins up to 3 rows, ties at 4
_workspaces = {}
_scratch_bufs = {}

# Act-order layers (g_idx a real permutation): sort the packed rows by group once per layer and
# run the sequential-group kernels on the sorted copy, gathering x through the permutation.
# Costs a second copy of qweight (K*N/2 bytes) per act-order layer; set to False to use the
# kernels that gather (scale, zero) through g_idx row by row instead.
actorder_repack = True


def _ptr(t):
    return 0 if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device) -> int:
    """Handle of torch's current stream on `device` (the raw getter skips building a Stream object per call)."""
    if _raw_stream is not None:
        return _raw_stream(device.index if device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(device).cuda_stream


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _device_ctx(device):
    """Context that makes `device` current for a launch; free when it already is (the usual case)."""
    if device.index is None or device.index == torch.cuda.current_device():
        return _NO_SWITCH
    return torch.cuda.device(device)


def _require(cond, msg):
    if not cond:
        raise ValueError(msg)


def _check_layer(qweight, qzeros, scales, g_idx, groupsize):
    """Validates a layer's tensors against each other; returns (device, K, N, G).  The verdict is kept on the
    qweight tensor object and reused while the same tensor objects (same storage, same dtypes) come back."""
    key = (id(qzeros), id(scales), id(g_idx), qweight.data_ptr(), qzeros.data_ptr(), scales.data_ptr(), scales.dtype,
           None if g_idx is None else g_idx.data_ptr(), groupsize if g_idx is None else None)
    cached = getattr(qweight, "_q4_layer", None)
    if cached is not None and cached[0] == key:
        return cached[1]
    result = _check_layer_uncached(qweight, qzeros, scales, g_idx, groupsize)
    try:
        qweight._q4_layer = (key, result)
    except AttributeError:          # tensor subclasses without a __dict__
        pass
    return result


def _check_layer_uncached(qweight, qzeros, scales, g_idx, groupsize):
    _require(qweight.is_cuda, "qweight must be on the GPU")
    dev = qweight.device
    _require(qweight.dtype == torch.int32 and qweight.dim() == 2, "qweight must be int32 [K/8, N]")
    _require(qzeros.dtype == torch.int32 and qzeros.dim() == 2, "qzeros must be int32 [G, N/8]")
    _require(scales.dtype == torch.float16 and scales.dim() == 2, "scales must be float16 [G, N]")
    K, N = qweight.shape[0] * 8, qweight.shape[1]
    G = scales.shape[0]
    _require(scales.shape[1] == N and tuple(qzeros.shape) == (G, N // 8),
             f"scales {tuple(scales.shape)} / qzeros {tuple(qzeros.shape)} do not match qweight {tuple(qweight.shape)}")
    for t in (qweight, qzeros, scales):
        _require(t.is_contiguous() and t.device == dev, "quantized tensors must be contiguous and on one device")
    if g_idx is not None:
        _require(g_idx.dtype == torch.int32 and g_idx.shape == (K,) and g_idx.is_contiguous() and g_idx.device == dev,
                 "g_idx must be a contiguous int32 [K] tensor on the same device")
    else:
        _require(groupsize is not None and groupsize > 0, "groupsize is required when g_idx is None")
    return dev, K, N, G


def classify_g_idx(g_idx, groupsize, G):
    """'seq' when g_idx[k] == k // groupsize for every k (the kernels then skip the gather),
    else 'gidx'.  Also validates 0 <= g_idx < G.  The verdict is cached on the tensor object
    together with its in-place version counter; the first call per tensor synchronises."""
    if g_idx is None:
        return "seq"
    key = (g_idx._version, int(groupsize or 0), G)
    cached = getattr(g_idx, "_q4_kind", None)
    if cached is not None and cached[0] == key:
        return cached[1]
    lo, hi = int(g_idx.min()), int(g_idx.max())
    if lo < 0 or hi >= G:
        raise ValueError(f"g_idx values must lie in [0, {G}); found [{lo}, {hi}]")
    kind = "gidx"
    if groupsize and groupsize > 0 and groupsize % 32 == 0:
        ref = torch.arange(g_idx.numel(), device=g_idx.device, dtype=torch.int32) // groupsize
        if bool(torch.equal(g_idx, ref)):
            kind = "seq"
    g_idx._q4_kind = (key, kind)
    return kind


def scales_fit_fused_dequant(scales):
    """True when every |scale| < 64: the GEMM kernels then form rn16(s*q) with one fused
    multiply-add on (1024 + q), which needs 1024*s to be finite.  Cached on the tensor like
    the g_idx verdict (first call per tensor synchronises).  Real GPTQ scales are ~1e-2."""
    key = scales._version
    cached = getattr(scales, "_q4_small", None)
    if cached is not None and cached[0] == key:
        return cached[1]
    ok = bool(torch.isfinite(scales).all()) and float(scales.abs().max()) < 64.0
    scales._q4_small = (key, ok)
    return ok


def _gemm_gidx_arg(g_idx, groupsize, G, K, scales):
    """Like _gidx_arg for the GEMM kernels; layers with huge scales are routed to the
    per-row-group path, whose dequant has no range restriction."""
    if scales_fit_fused_dequant(scales) and not (g_idx is None and int(groupsize) % 64 != 0):
        return _gidx_arg(g_idx, groupsize, G, need_multiple=64) + (g_idx,)
    if g_idx is None:            # sequential groups the tiled kernels do not take as such (group size not a multiple of 64)
        g_idx = (torch.arange(K, device=scales.device, dtype=torch.int32) // int(groupsize)).contiguous()
    return g_idx.data_ptr(), int(groupsize or 0), g_idx


def sorted_layer(qweight, g_idx, G):
    """(perm, inv_perm, qweight_sorted, groupsize) for an act-order layer whose groups all own
    exactly K/G rows (what GPTQ's act-order produces), else None.  perm[p] is the original index of
    sorted row p.  Built once per (g_idx, qweight) pair and cached on the g_idx tensor object."""
    K, N = qweight.shape[0] * 8, qweight.shape[1]
    key = (g_idx._version, qweight._version, qweight.data_ptr())
    cached = getattr(g_idx, "_q4_sorted", None)
    if cached is not None and cached[0] == key:
        return cached[1]
    plan = None
    if K % G == 0 and (K // G) % 64 == 0:
        counts = torch.bincount(g_idx.long(), minlength=G)
        if bool((counts == K // G).all()):
            perm = torch.argsort(g_idx.long(), stable=True).to(torch.int32).contiguous()
            inv = torch.empty_like(perm)
            inv[perm.long()] = torch.arange(K, device=perm.device, dtype=torch.int32)
            qs = torch.empty_like(qweight)
            with _device_ctx(qweight.device):
                rc = _lib.lib().q4_permute_rows(qweight.data_ptr(), perm.data_ptr(), qs.data_ptr(), K, N,
                                                _stream(qweight.device))
            _lib.check(rc, "q4_permute_rows")
            plan = (perm, inv, qs, K // G)
    g_idx._q4_sorted = (key, plan)
    return plan


def permute_cols(x, idx):
    """out fp16 [M, K] with out[m, p] = x[m, idx[p]] (idx int32 [K]): the activations of an act-order layer gathered through
    the row sort of its weights, or a grad_input gathered back through the inverse permutation."""
    M, K = x.shape
    if M == 0 or K % 8 or K > 32768 or x.data_ptr() % 16:
        return x.index_select(1, idx)
    out = torch.empty_like(x)
    with _device_ctx(x.device):
        rc = _lib.lib().q4_permute_cols_f16(x.data_ptr(), idx.data_ptr(), out.data_ptr(), M, K, _stream(x.device))
    _lib.check(rc, "q4_permute_cols_f16")
    return out


def _actorder_plan(qweight, scales, g_idx, groupsize, G):
    """The sorted-copy plan when this call should use it, else None."""
    if g_idx is None or not actorder_repack:
        return None
    if classify_g_idx(g_idx, groupsize, G) != "gidx" or not scales_fit_fused_dequant(scales):
        return None
    return sorted_layer(qweight, g_idx, G)


class _LayerInfo:
    """What the content-dependent checks decided for one layer's tensors: how the GEMV and the GEMM kernels are to
    be called (g_idx tensor or None for sequential groups, group size) and the sorted-rows plan of an act-order layer."""
    __slots__ = ("dev", "K", "N", "G", "gemv_gidx", "gemv_gs", "gemm", "plan", "_src")

    def gemm_args(self):
        """(g_idx tensor or None, group size) for the tiled kernels; decided on the first product above 16 rows."""
        if self.gemm is None:
            g_idx, groupsize, scales = self._src
            gp, gs, keep = _gemm_gidx_arg(g_idx, groupsize, self.G, self.K, scales)
            self.gemm = (None if gp == 0 else keep, gs)
        return self.gemm


def _layer_info(qweight, qzeros, scales, g_idx, groupsize):
    """_LayerInfo of these tensors.  Kept on the qweight tensor object and reused while the very same tensor objects
    come back with unchanged in-place version counters: a handful of identity and integer comparisons per call.
    (Writes through `.data` do not bump the counters: call `invalidate` after such a write.)"""
    gver = -1 if g_idx is None else g_idx._version
    c = getattr(qweight, "_q4_info", None)
    if (c is not None and c[0] is qzeros and c[1] is scales and c[2] is g_idx and c[3] == groupsize
            and c[4] == qweight._version and c[5] == qzeros._version and c[6] == scales._version and c[7] == gver
            and c[8] == actorder_repack):
        return c[9]
    info = _LayerInfo()
    info.dev, info.K, info.N, info.G = _check_layer_uncached(qweight, qzeros, scales, g_idx, groupsize)
    info.plan = _actorder_plan(qweight, scales, g_idx, groupsize, info.G)
    info._src = (g_idx, groupsize, scales)
    info.gemm = None
    if info.plan is not None:
        info.gemv_gidx, info.gemv_gs = None, info.plan[3]
        info.gemm = (None, info.plan[3])
    else:
        gp, gs = _gidx_arg(g_idx, groupsize, info.G)
        info.gemv_gidx, info.gemv_gs = (None if gp == 0 else g_idx), gs
    try:
        qweight._q4_info = (qzeros, scales, g_idx, groupsize, qweight._version, qzeros._version, scales._version, gver,
                            actorder_repack, info)
    except AttributeError:          # tensor subclasses without a __dict__
        pass
    return info


def invalidate(*tensors_or_modules):
    """Forget what was cached about these tensors (or about every tensor of these modules): the layer verdicts,
    the g_idx classification, the scale-range check and the sorted copy of an act-order layer.  Needed only after
    writing packed tensors through `.data` (which does not bump the version counter the caches are keyed on)."""
    for obj in tensors_or_modules:
        items = [obj] if isinstance(obj, torch.Tensor) else [t for _, t in obj.named_buffers()] + list(obj.parameters())
        for t in items:
            for name in ("_q4_info", "_q4_layer", "_q4_kind", "_q4_small", "_q4_sorted", "_q4_zero"):
                if hasattr(t, name):
                    try:
                        delattr(t, name)
                    except AttributeError:
                        pass


def _shape_arg(out_shape):
    return None if out_shape is None else [int(d) for d in out_shape]


def _gidx_arg(g_idx, groupsize, G, need_multiple=32):
    """Returns (pointer-or-0, groupsize) to hand to the C ABI."""
    if g_idx is None:
        _require(groupsize % need_multiple == 0, f"groupsize must be a multiple of {need_multiple} without g_idx")
        return 0, int(groupsize)
    kind = classify_g_idx(g_idx, groupsize, G)
    if kind == "seq" and groupsize % need_multiple == 0:
        return 0, int(groupsize)
    return g_idx.data_ptr(), int(groupsize or 0)


def _workspace(device, nbytes):
    key = (device.index, _stream(device))
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.zeros(max(nbytes, 1 << 22), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def workspaces_are_zero():
    """True when the GEMV's split-K accumulators cached for every (device, stream) are all zero, as every completed
    call leaves them (synchronises; for tests and debugging).  `Q4_CHECK_WORKSPACE=1` in the environment makes the
    compiled host binding check this on entry of every GEMV."""
    ok = all(int(ws.view(torch.int32).abs().max()) == 0 for ws in _workspaces.values())
    return ok and (_host is None or _host.workspaces_are_zero())


def reset_workspaces():
    """Zeroes the cached GEMV accumulators (after a run that was cut short inside a GEMV)."""
    for ws in _workspaces.values():
        ws.zero_()
    if _host is not None:
        _host.reset_workspaces()


def _scratch(device, nbytes):
    """Uninitialised scratch (partial sums); kept apart from the zero-on-entry split-K workspace."""
    key = (device.index, _stream(device))
    buf = _scratch_bufs.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(nbytes, 1 << 22), dtype=torch.uint8, device=device)
        _scratch_bufs[key] = buf
    return buf


def _gemm_scratch(L, device, fwd, M, K, N):
    """(pointer, bytes) of the split-K scratch the GEMM would like for this shape, or (None, 0)."""
    nbytes = L.q4_gemm_workspace_bytes(fwd, M, K, N)
    if nbytes == 0:
        return None, 0
    buf = _scratch(device, nbytes)
    return buf.data_ptr(), buf.numel()


def _out_shape(out_shape, rows, cols):
    if out_shape is None:
        return (rows, cols)
    out_shape = tuple(out_shape)
    n = 1
    for d in out_shape:
        n *= d
    _require(len(out_shape) >= 1 and out_shape[-1] == cols and n == rows * cols,
             f"out_shape {out_shape} does not hold {rows} rows of {cols}")
    return out_shape


def _flat_half(x, K, dev, what):
    _require(x.is_cuda and x.device == dev, f"{what} must be on {dev}")
    _require(x.shape[-1] == K, f"{what} last dimension {x.shape[-1]} != {K}")
    x2 = x.reshape(-1, K)
    if x2.dtype != torch.float16:
        x2 = x2.half()
    return x2.contiguous()


# ------------------------------------------------------------------------------- operators
def dequant(qweight, qzeros, scales, g_idx=None, groupsize=None, out=None):
    """W fp16 [K, N], bit-exact with vecquant4recons_v2 (quant_cuda_kernel.cu:1127-1153)."""
    dev, K, N, G = _check_layer(qweight, qzeros, scales, g_idx, groupsize)
    gp, gs = _gidx_arg(g_idx, groupsize, G, need_multiple=8)
    if _host is not None:
        return _host.dequant(qweight, qzeros, scales, None if gp == 0 else g_idx, gs, out)
    if out is None:
        out = torch.empty((K, N), dtype=torch.float16, device=dev)
    _require(out.dtype == torch.float16 and tuple(out.shape) == (K, N) and out.is_contiguous() and out.device == dev,
             "out must be a contiguous float16 [K, N] tensor on the same device")
    with _device_ctx(dev):
        rc = _lib.lib().q4_dequant_f16(qweight.data_ptr(), qzeros.data_ptr(), scales.data_ptr(), gp, gs,
                                       out.data_ptr(), K, N, G, _stream(dev))
    _lib.check(rc, "q4_dequant_f16")
    return out


def dequant_f32(qweight, qzeros, scales, g_idx=None, groupsize=None, out=None):
    """W fp32 [K, N] from fp32 scales: the float instantiation of vecquant4recons_v2
    (quant_cuda_kernel.cu:1126-1152 through the dispatch at :1173-1181).  zero = rn32(s * (z + 1)),
    W = fma(s, q, -zero), the contraction the reference's default build applies."""
    _require(scales.dtype == torch.float32, "scales must be float32 [G, N]")
    _require(qweight.is_cuda and qweight.dtype == torch.int32 and qweight.dim() == 2, "qweight must be int32 [K/8, N] on the GPU")
    dev = qweight.device
    K, N = qweight.shape[0] * 8, qweight.shape[1]
    _require(scales.dim() == 2 and scales.shape[1] == N, "scales must be float32 [G, N]")
    G = scales.shape[0]
    _require(qzeros.dtype == torch.int32 and tuple(qzeros.shape) == (G, N // 8), "qzeros must be int32 [G, N/8]")
    for t in (qweight, qzeros, scales):
        _require(t.is_contiguous() and t.device == dev, "quantized tensors must be contiguous and on one device")
    if g_idx is not None:
        _require(g_idx.dtype == torch.int32 and g_idx.shape == (K,) and g_idx.is_contiguous() and g_idx.device == dev,
                 "g_idx must be a contiguous int32 [K] tensor on the same device")
    gp, gs = _gidx_arg(g_idx, groupsize, G, need_multiple=8)
    if out is None:
        out = torch.empty((K, N), dtype=torch.float32, device=dev)
    _require(out.dtype == torch.float32 and tuple(out.shape) == (K, N) and out.is_contiguous() and out.device == dev,
             "out must be a contiguous float32 [K, N] tensor on the same device")
    with _device_ctx(dev):
        rc = _lib.lib().q4_dequant_f32(qweight.data_ptr(), qzeros.data_ptr(), scales.data_ptr(), gp, gs,
                                       out.data_ptr(), K, N, G, _stream(dev))
    _lib.check(rc, "q4_dequant_f32")
    return out


def dequant_v1(qweight, scales, zeros, out=None):
    """W fp16 [K, N] of a v1 layer (per-column fp16 scale and zero), bit-exact with vecquant4recons_v1
    (quant_cuda_kernel.cu:1076-1097)."""
    _require(qweight.is_cuda and qweight.dtype == torch.int32 and qweight.dim() == 2 and qweight.is_contiguous(),
             "qweight must be a contiguous int32 [K/8, N] CUDA tensor")
    dev = qweight.device
    K, N = qweight.shape[0] * 8, qweight.shape[1]
    s1 = scales.reshape(-1)
    z1 = zeros.reshape(-1)
    _require(s1.numel() == N and z1.numel() == N and s1.device == dev and z1.device == dev,
             "v1 scales and zeros hold one value per column")
    s1 = s1 if s1.dtype == torch.float16 else s1.half()
    z1 = z1 if z1.dtype == torch.float16 else z1.half()
    s1, z1 = s1.contiguous(), z1.contiguous()
    _require(N % 64 == 0, "N must be a multiple of 64")
    if out is None:
        out = torch.empty((K, N), dtype=torch.float16, device=dev)
    _require(out.dtype == torch.float16 and tuple(out.shape) == (K, N) and out.is_contiguous() and out.device == dev,
             "out must be a contiguous float16 [K, N] tensor on the same device")
    with _device_ctx(dev):
        rc = _lib.lib().q4_dequant_v1_f16(qweight.data_ptr(), s1.data_ptr(), z1.data_ptr(), out.data_ptr(), K, N,
                                          _stream(dev))
    _lib.check(rc, "q4_dequant_v1_f16")
    return out


def gemv_v1(x, qweight, scales, zeros, out=None, accumulate=False, out_shape=None):
    """y fp16 [M, N] = x [M, K] @ W for a v1 layer (per-column fp16 scale and zero), M <= 16: the decode product
    of vecquant4matmul_v1_faster (quant_cuda_kernel.cu:1244-1302) with fp32 accumulation."""
    _require(qweight.is_cuda and qweight.dtype == torch.int32 and qweight.dim() == 2 and qweight.is_contiguous(),
             "qweight must be a contiguous int32 [K/8, N] CUDA tensor")
    dev = qweight.device
    K, N = qweight.shape[0] * 8, qweight.shape[1]
    s1, z1 = scales.reshape(-1), zeros.reshape(-1)
    _require(s1.numel() == N and z1.numel() == N and s1.device == dev and z1.device == dev,
             "v1 scales and zeros hold one value per column")
    s1 = (s1 if s1.dtype == torch.float16 else s1.half()).contiguous()
    z1 = (z1 if z1.dtype == torch.float16 else z1.half()).contiguous()
    _require(K % 32 == 0 and N % 64 == 0, "K must be a multiple of 32 and N of 64")
    x2 = _flat_half(x, K, dev, "x")
    M = x2.shape[0]
    if M == 0 and out is None:                              # empty batch: nothing to launch
        return torch.empty(_out_shape(out_shape, 0, N), dtype=torch.float16, device=dev)
    _require(1 <= M <= MAX_GEMV_ROWS, f"gemv handles 1..{MAX_GEMV_ROWS} rows, got {M}")
    if out is None:
        _require(not accumulate, "accumulate needs an output tensor")
        out = torch.empty(_out_shape(out_shape, M, N), dtype=torch.float16, device=dev)
    _require(out.dtype == torch.float16 and out.numel() == M * N and out.shape[-1] == N and out.is_contiguous()
             and out.device == dev, "out must be a contiguous float16 [..., N] tensor with M rows on the same device")
    L = _lib.lib()
    with _device_ctx(dev):
        ws = _workspace(dev, L.q4_gemv_workspace_bytes(M, K, N))
        rc = L.q4_gemv_v1_f16(x2.data_ptr(), qweight.data_ptr(), s1.data_ptr(), z1.data_ptr(), out.data_ptr(),
                              int(bool(accumulate)), M, K, N, ws.data_ptr(), ws.numel(), _stream(dev))
    _lib.check(rc, "q4_gemv_v1_f16")
    return out


def dequant2(qweight, qzeros, scales, g_idx=None, groupsize=None, out=None):
    """W fp16 [K, N] of a 2-bit v2 layer (qweight [K/16, N], qzeros [G, N/16]), bit-exact with
    vecquant2recons_v2 (quant_cuda_kernel.cu:1185-1211)."""
    for name, tns, dt in (("qweight", qweight, torch.int32), ("qzeros", qzeros, torch.int32), ("scales", scales, torch.float16)):
        _require(tns.is_cuda and tns.dtype == dt and tns.dim() == 2 and tns.is_contiguous(),
                 f"{name} must be a contiguous 2-D {dt} CUDA tensor")
    dev = qweight.device
    K, N = qweight.shape[0] * 16, qweight.shape[1]
    G = scales.shape[0]
    _require(N % 64 == 0 and tuple(scales.shape) == (G, N) and tuple(qzeros.shape) == (G, N // 16)
             and qzeros.device == dev and scales.device == dev, "2-bit layer shapes do not match")
    gp, gs = 0, int(groupsize or -(-K // G))
    if g_idx is not None:
        _require(g_idx.dtype == torch.int32 and g_idx.numel() == K and g_idx.device == dev and g_idx.is_contiguous(),
                 "g_idx must be a contiguous int32 [K] tensor on the same device")
        if classify_g_idx(g_idx, gs, G) != "seq" or gs % 16 != 0:
            gp = g_idx.data_ptr()
    if out is None:
        out = torch.empty((K, N), dtype=torch.float16, device=dev)
    _require(out.dtype == torch.float16 and tuple(out.shape) == (K, N) and out.is_contiguous() and out.device == dev,
             "out must be a contiguous float16 [K, N] tensor on the same device")
    with _device_ctx(dev):
        rc = _lib.lib().q4_dequant2_f16(qweight.data_ptr(), qzeros.data_ptr(), scales.data_ptr(), gp, gs,
                                        out.data_ptr(), K, N, G, _stream(dev))
    _lib.check(rc, "q4_dequant2_f16")
    return out


def gemv(x, qweight, qzeros, scales, g_idx=None, groupsize=None, out=None, accumulate=False, out_shape=None):
    """y fp16 [M, N] = x [M, K] @ W for M <= 16 (decode).  `out_shape` (same number of elements)
    lets the result be allocated with the caller's leading dimensions instead of being a view."""
    if _host is not None:
        info = _layer_info(qweight, qzeros, scales, g_idx, groupsize)
        if info.plan is None:
            return _host.gemv(x, qweight, qzeros, scales, info.gemv_gidx, info.gemv_gs, out, bool(accumulate),
                              _shape_arg(out_shape))
    dev, K, N, G = _check_layer(qweight, qzeros, scales, g_idx, groupsize)
    x2 = _flat_half(x, K, dev, "x")
    M = x2.shape[0]
    if M == 0 and out is None:                              # empty batch: nothing to launch
        return torch.empty(_out_shape(out_shape, 0, N), dtype=torch.float16, device=dev)
    _require(1 <= M <= MAX_GEMV_ROWS, f"gemv handles 1..{MAX_GEMV_ROWS} rows, got {M}")
    if out is None:
        _require(not accumulate, "accumulate needs an output tensor")
        out = torch.empty(_out_shape(out_shape, M, N), dtype=torch.float16, device=dev)
    _require(out.dtype == torch.float16 and out.numel() == M * N and out.shape[-1] == N and out.is_contiguous()
             and out.device == dev, "out must be a contiguous float16 [..., N] tensor with M rows on the same device")
    L = _lib.lib()
    nbytes = L.q4_gemv_workspace_bytes(M, K, N)
    plan = _actorder_plan(qweight, scales, g_idx, groupsize, G)
    if plan is not None and M <= MAX_GEMV_SORTED_ROWS and K >= 1024 and M * (2 * K + 4096) <= 65536:     # rows fit in LDS
        # sorted copy of the packed rows; the kernel gathers x through the permutation itself
        perm, _, qweight, gs_sorted = plan
        with _device_ctx(dev):
            ws = _workspace(dev, nbytes)
            rc = L.q4_gemv_sorted_f16(x2.data_ptr(), qweight.data_ptr(), qzeros.data_ptr(), scales.data_ptr(),
                                      perm.data_ptr(), gs_sorted, out.data_ptr(), int(bool(accumulate)), M, K, N, G,
                                      ws.data_ptr(), ws.numel(), _stream(dev))
        _lib.check(rc, "q4_gemv_sorted_f16")
        return out
    if plan is not None:
        perm, _, qweight, gs_sorted = plan
        x2 = permute_cols(x2, perm)
        gp, gs = 0, gs_sorted
    else:
        gp, gs = _gidx_arg(g_idx, groupsize, G)
    with _device_ctx(dev):
        ws = _workspace(dev, nbytes)
        rc = L.q4_gemv_f16(x2.data_ptr(), qweight.data_ptr(), qzeros.data_ptr(), scales.data_ptr(), gp, gs,
                           out.data_ptr(), int(bool(accumulate)), M, K, N, G, ws.data_ptr(), ws.numel(), _stream(dev))
    _lib.check(rc, "q4_gemv_f16")
    return out


def gemv_grouped(xs, layers, groupsize, outs=None, accumulate=False):
    """[x_i @ W_i] for up to 4 layers that share the number of rows (<= 16), K and the group size, in ONE launch
    over the layers' own tensors (no concatenated copy): q|k|v or gate|up of a decoder block at decode time.
    `xs` is one activation tensor shared by all layers or a list with one per layer; `layers` a list of
    (qweight, qzeros, scales) or (qweight, qzeros, scales, g_idx) with sequential groups; returns the list of
    outputs ([M, N_i] fp16 each).  The reference concatenates the packed tensors instead
    (model_attn_mlp_patch.py:88-100, 180-190)."""
    n = len(layers)
    _require(1 <= n <= _lib.MAX_GEMV_GROUP, f"gemv_grouped takes 1..{_lib.MAX_GEMV_GROUP} layers")
    if isinstance(xs, torch.Tensor):
        xs = [xs] * n
    _require(len(xs) == n, "one activation tensor per layer (or a single shared one)")
    if _host is not None:
        for lay in layers:
            info = _layer_info(lay[0], lay[1], lay[2], lay[3] if len(lay) > 3 else None, groupsize)
            _require(info.plan is None and info.gemv_gidx is None, "gemv_grouped needs sequential groups (no act-order)")
        return _host.gemv_grouped(list(xs), [(lay[0], lay[1], lay[2]) for lay in layers], int(groupsize),
                                  None if outs is None else list(outs), bool(accumulate))
    dev = K = M = None
    desc = (_lib.GemvLayer * n)()
    keep, shapes = [], []
    flat = {}
    for i, (x, lay) in enumerate(zip(xs, layers)):
        qweight, qzeros, scales = lay[0], lay[1], lay[2]
        g_idx = lay[3] if len(lay) > 3 else None
        d, k, N, G = _check_layer(qweight, qzeros, scales, g_idx, groupsize)
        _require(g_idx is None or classify_g_idx(g_idx, groupsize, G) == "seq",
                 "gemv_grouped needs sequential groups (no act-order)")
        if dev is None:
            dev, K = d, k
        _require(d == dev and k == K, "grouped layers must share the device and K")
        x2 = flat.get(id(x))
        if x2 is None:
            x2 = flat[id(x)] = _flat_half(x, K, dev, "x")
        if M is None:
            M = x2.shape[0]
        _require(x2.shape[0] == M, "grouped layers must share the number of rows")
        keep.append(x2)
        shapes.append(N)
        desc[i].x, desc[i].qweight, desc[i].qzeros, desc[i].scales, desc[i].N = (
            x2.data_ptr(), qweight.data_ptr(), qzeros.data_ptr(), scales.data_ptr(), N)
    _require(groupsize % 32 == 0, "groupsize must be a multiple of 32")
    _require(1 <= M <= MAX_GEMV_ROWS, f"gemv handles 1..{MAX_GEMV_ROWS} rows, got {M}")
    if outs is None:
        _require(not accumulate, "accumulate needs output tensors")
        outs = [torch.empty((M, N), dtype=torch.float16, device=dev) for N in shapes]
    _require(len(outs) == n, "one output per layer")
    for i, (o, N) in enumerate(zip(outs, shapes)):
        _require(o.dtype == torch.float16 and o.numel() == M * N and o.shape[-1] == N and o.is_contiguous()
                 and o.device == dev, "outputs must be contiguous float16 [..., N_i] tensors with M rows on the same device")
        desc[i].y = o.data_ptr()
    L = _lib.lib()
    with _device_ctx(dev):
        ws = _workspace(dev, L.q4_gemv_grouped_workspace_bytes(M, sum(shapes)))
        rc = L.q4_gemv_grouped_f16(desc, n, int(groupsize), int(bool(accumulate)), M, K, ws.data_ptr(), ws.numel(),
                                   _stream(dev))
    _lib.check(rc, "q4_gemv_grouped_f16")
    return list(outs)


def mlp_decode_applicable(M, H, I, groupsize):
    """Shapes `mlp_decode` takes (chunks of 128 reduction rows inside one quantization group on both sides)."""
    return (1 <= M <= MAX_GEMV_ROWS and groupsize and groupsize % 128 == 0 and H % 128 == 0 and I % 128 == 0
            and H >= 128 and I >= 128)


def mlp_decode(x, gate, up, down, groupsize, intermediates=False, out_shape=None):
    """y fp16 [M, H] = down(silu(gate(x)) * up(x)) for M <= 16 rows in ONE launch: the decode step of the reference's
    QuantLlamaMLP.forward (model_attn_mlp_patch.py:224-228).  `gate`, `up` (H -> I) and `down` (I -> H) are
    (qweight, qzeros, scales) or (qweight, qzeros, scales, g_idx) of layers with sequential groups and no bias.
    With `intermediates` returns (y, gate(x), up(x))."""
    _require(_host is not None, "mlp_decode needs the compiled host binding (_q4_host)")
    lays = []
    for lay in (gate, up, down):
        info = _layer_info(lay[0], lay[1], lay[2], lay[3] if len(lay) > 3 else None, groupsize)
        _require(info.plan is None and info.gemv_gidx is None, "mlp_decode needs sequential groups (no act-order)")
        lays.append((lay[0], lay[1], lay[2]))
    res = _host.mlp_decode(x, lays[0], lays[1], lays[2], int(groupsize), bool(intermediates), _shape_arg(out_shape))
    return tuple(res) if intermediates else res[0]


def gemv_grouped_prepared(x, layers, groupsize):
    """gemv_grouped for callers that already know the layers qualify (sequential groups, fp16 scales: the module
    groups of model_attn_mlp_patch establish that once): straight to the compiled binding, which still checks shapes,
    dtypes and devices.  `layers`: list of (qweight, qzeros, scales)."""
    return _host.gemv_grouped([x] * len(layers), layers, groupsize, None, False)


def mlp_decode_prepared(x, gate, up, down, groupsize, out_shape):
    """mlp_decode under the same premise as gemv_grouped_prepared."""
    return _host.mlp_decode(x, gate, up, down, groupsize, False, out_shape)[0]


def mlp_decode_gave_up():
    """True when a device-side wait of some `mlp_decode` launch ran into its poll limit (synchronises)."""
    return bool(_host is not None and _host.mlp_decode_gave_up())


def _adapter_dtype_flag(w, what):
    _require(w.dtype in (torch.float16, torch.float32), f"{what} must be float16 or float32")
    return int(w.dtype == torch.float32)


def _lora_pair(la, lb, rows, cols, dev):
    """la: [rows, R] fp16 contiguous; lb: [R, cols] fp16 or fp32 with any (positive) strides."""
    if la is None and lb is None:
        return None, None, 0, 0, 0, 0
    _require(la is not None and lb is not None, "both LoRA operands are required")
    R = la.shape[-1]
    _require(la.dtype == torch.float16, "the rank-R activation operand must be float16")
    is_f32 = _adapter_dtype_flag(lb, "the adapter matrix")
    _require(tuple(la.shape) == (rows, R) and tuple(lb.shape) == (R, cols), "LoRA operand shapes do not match")
    _require(R % 8 == 0 and 8 <= R <= 64, "LoRA rank must be a multiple of 8 in [8, 64] for the fused path")
    _require(la.is_contiguous() and la.device == dev and lb.device == dev, "LoRA operands must be on the same device")
    sr, sc = lb.stride()
    _require(sr >= 1 and sc >= 1, "the adapter matrix must have positive strides")
    return la, lb, R, int(sr), int(sc), is_f32


def gemm_fwd(x, qweight, qzeros, scales, g_idx=None, groupsize=None, bias=None, xa=None, lora_bt=None,
             lora_scale=1.0, out_shape=None):
    """y fp16 [M, N] = x @ W (+ bias) (+ lora_scale * xa @ lora_bt), W dequantized tile by tile in LDS.
    `lora_bt` is the adapter matrix as an [R, N] fp16/fp32 view with any strides (e.g. `lora_B.weight.t()`)."""
    if _host is not None:
        info = _layer_info(qweight, qzeros, scales, g_idx, groupsize)
        if info.plan is None:
            gi, gs = info.gemm_args()
            return _host.gemm_fwd(x, qweight, qzeros, scales, gi, gs, bias, xa, lora_bt,
                                  float(lora_scale), _shape_arg(out_shape))
        if info.K % 8 == 0 and info.K <= 32768:
            # act-order layer with a sorted copy of its rows: x gathered through the sort, then sequential groups
            perm, _, qsorted, gs_sorted = info.plan
            return _host.gemm_fwd(x, qsorted, qzeros, scales, None, gs_sorted, bias, xa, lora_bt,
                                  float(lora_scale), _shape_arg(out_shape), perm)
    dev, K, N, G = _check_layer(qweight, qzeros, scales, g_idx, groupsize)
    x2 = _flat_half(x, K, dev, "x")
    M = x2.shape[0]
    if M == 0:                                               # empty batch: nothing to launch
        return torch.empty(_out_shape(out_shape, 0, N), dtype=torch.float16, device=dev)
    if bias is not None:
        _require(bias.dtype == torch.float16 and tuple(bias.shape) == (N,) and bias.is_contiguous()
                 and bias.device == dev, "bias must be a contiguous float16 [N] tensor on the same device")
    xa, lora_bt, R, sr, sc, f32 = _lora_pair(xa, lora_bt, M, N, dev)
    plan = _actorder_plan(qweight, scales, g_idx, groupsize, G)
    if plan is not None:
        perm, _, qweight, gs_sorted = plan
        x2 = permute_cols(x2, perm)
        gp, gs = 0, gs_sorted
    else:
        gp, gs, _keepalive = _gemm_gidx_arg(g_idx, groupsize, G, K, scales)
    out = torch.empty(_out_shape(out_shape, M, N), dtype=torch.float16, device=dev)
    L = _lib.lib()
    with _device_ctx(dev):
        wp, wn = _gemm_scratch(L, dev, 1, M, K, N)
        rc = L.q4_gemm_fwd_f16(x2.data_ptr(), qweight.data_ptr(), qzeros.data_ptr(), scales.data_ptr(),
                               gp, gs, _ptr(bias), _ptr(xa), _ptr(lora_bt), sr, sc, f32, float(lora_scale), R,
                               out.data_ptr(), M, K, N, G, wp, wn, _stream(dev))
    _lib.check(rc, "q4_gemm_fwd_f16")
    return out


def gemm_grouped_applicable(fwd, M, K, Ns):
    """True when gemm_grouped_fwd / gemm_grouped_bwd_dx take this shape (2..4 layers, more than 128 rows, enough tiles
    for one launch); the layers must also have sequential groups and scales below 64 (checked by those calls)."""
    n = len(Ns)
    if not 2 <= n <= 4:
        return False
    arr = (ctypes.c_int * n)(*[int(v) for v in Ns])
    return bool(_lib.lib().q4_gemm_grouped_applicable(int(bool(fwd)), n, int(M), int(K), arr))


def _group_layer_ok(lay, groupsize):
    info = _layer_info(lay[0], lay[1], lay[2], None, groupsize)
    return info.plan is None and info.gemm_args()[0] is None


def gemm_grouped_fwd(x, layers, groupsize):
    """[x @ W_i (+ bias_i) (+ scale_i * xa_i @ lora_bt_i)] for 2..4 layers that share x, K and the group size, in ONE
    launch over the layers' own tensors (q|k|v or gate|up of a decoder block above 128 rows).  `layers`: list of
    (qweight, qzeros, scales, bias | None, xa | None, lora_bt | None, lora_scale).  Returns the [M, N_i] outputs."""
    _require(_host is not None, "gemm_grouped_fwd needs the compiled host binding (_q4_host)")
    for lay in layers:
        _require(_group_layer_ok(lay, groupsize), "gemm_grouped_fwd needs sequential groups and scales below 64")
    return _host.gemm_grouped_fwd(x, [(l[0], l[1], l[2], l[3], l[4], l[5], float(l[6]), None) for l in layers], int(groupsize))


def gemm_grouped_bwd_dx(dys, layers, groupsize, out_shape=None):
    """dx = sum_i (dy_i @ W_i^T + mask_i * scale_i * dyb_i @ lora_a_i): the grad-inputs of 2..4 layers that share their
    input, summed, in one launch and one ordered reduction.  `layers`: list of (qweight, qzeros, scales, dyb | None,
    lora_a | None, lora_scale, dropout (seed, p) | None)."""
    _require(_host is not None, "gemm_grouped_bwd_dx needs the compiled host binding (_q4_host)")
    for lay in layers:
        _require(_group_layer_ok(lay, groupsize), "gemm_grouped_bwd_dx needs sequential groups and scales below 64")
    return _host.gemm_grouped_bwd_dx(list(dys), [(l[0], l[1], l[2], None, l[3], l[4], float(l[5]),
                                                  None if l[6] is None else (int(l[6][0]), float(l[6][1]))) for l in layers],
                                     int(groupsize), _shape_arg(out_shape))


def _drop_arg(dropout):
    """(seed, p) -> ctypes descriptor (kept alive by the caller for the duration of the call), or None."""
    if dropout is None:
        return None
    seed, p = dropout
    p = float(p)
    _require(0.0 <= p < 1.0, "dropout probability must be in [0, 1)")
    if p == 0.0:
        return None
    seed = int(seed)
    return _lib.Dropout(seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF, p)


def _drop_ref(d):
    return None if d is None else ctypes.byref(d)


def dropout_scale(p):
    """What the kernels multiply the surviving elements by: 1 / (1 - round(p * 32768) / 32768)."""
    return float(_lib.lib().q4_dropout_scale(float(p)))


def dropout_keep_mask(M, C, seed, p, device="cuda"):
    """uint8 [M, C]: 1 where the counter-based dropout of (seed, p) keeps element (m, c), the mask that lora_down,
    lora_grad and gemm_bwd_dx regenerate internally when given dropout=(seed, p)."""
    dev = torch.device(device)
    keep = torch.empty((M, C), dtype=torch.uint8, device=dev)
    seed = int(seed)
    d = _lib.Dropout(seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF, float(p))
    with _device_ctx(dev):
        rc = _lib.lib().q4_dropout_keep_u8(keep.data_ptr(), M, C, ctypes.byref(d), _stream(dev))
    _lib.check(rc, "q4_dropout_keep_u8")
    return keep


def masked_adapter_term(dyb, lora_a, lora_scale, dropout):
    """fp16 [M, K]: mask/(1-p) * lora_scale * dyb @ lora_a under the counter-based mask of dropout=(seed, p):
    the adapter's share of grad_input for the routes that do not run the fused backward kernel."""
    M, K = dyb.shape[0], lora_a.shape[1]
    term = torch.mm(dyb * (float(lora_scale) * dropout_scale(dropout[1])), lora_a.to(torch.float16))
    return term.mul_(dropout_keep_mask(M, K, dropout[0], dropout[1], dyb.device))


def gemm_bwd_dx(dy, qweight, qzeros, scales, g_idx=None, groupsize=None, dyb=None, lora_a=None, lora_scale=1.0,
                out_shape=None, dropout=None):
    """dx fp16 [M, K] = dy [M, N] @ W^T (+ lora_scale * dyb @ lora_a); lora_a is an [R, K] view.
    dropout=(seed, p): the adapter term is masked like dropout(x) (gradient of lora_B(lora_A(dropout(x))))."""
    if _host is not None:
        info = _layer_info(qweight, qzeros, scales, g_idx, groupsize)
        if info.plan is None:
            gi, gs = info.gemm_args()
            return _host.gemm_bwd_dx(dy, qweight, qzeros, scales, gi, gs, dyb, lora_a,
                                     float(lora_scale), _shape_arg(out_shape),
                                     None if dropout is None else (int(dropout[0]), float(dropout[1])))
        if dyb is None and info.K % 8 == 0 and info.K <= 32768:
            # act-order layer, no adapter term: grad_input in sorted order, gathered back through the inverse permutation
            _, inv, qsorted, gs_sorted = info.plan
            return _host.gemm_bwd_dx(dy, qsorted, qzeros, scales, None, gs_sorted, None, None, 1.0,
                                     _shape_arg(out_shape), None, inv)
    dev, K, N, G = _check_layer(qweight, qzeros, scales, g_idx, groupsize)
    dy2 = _flat_half(dy, N, dev, "grad_output")
    M = dy2.shape[0]
    if M == 0:
        return torch.empty(_out_shape(out_shape, 0, K), dtype=torch.float16, device=dev)
    plan = _actorder_plan(qweight, scales, g_idx, groupsize, G)
    if plan is not None:
        # dx comes out in sorted row order and is scattered back; the adapter matrix [R, K] is gathered too
        perm, inv, qs, gs_sorted = plan
        if dropout is not None and dyb is not None:
            # the mask is indexed by the ORIGINAL column: add the masked adapter term after the scatter
            dx_sorted = gemm_bwd_dx(dy2, qs, qzeros, scales, None, gs_sorted)
            dx = permute_cols(dx_sorted, inv)
            return dx.add_(masked_adapter_term(dyb, lora_a, lora_scale, dropout)).reshape(_out_shape(out_shape, M, K))
        la_sorted = None if lora_a is None else lora_a.index_select(1, perm)
        dx_sorted = gemm_bwd_dx(dy2, qs, qzeros, scales, None, gs_sorted, dyb=dyb, lora_a=la_sorted, lora_scale=lora_scale)
        return permute_cols(dx_sorted, inv).reshape(_out_shape(out_shape, M, K))
    dyb, lora_a, R, sr, sc, f32 = _lora_pair(dyb, lora_a, M, K, dev)
    gp, gs, _keepalive = _gemm_gidx_arg(g_idx, groupsize, G, K, scales)
    out = torch.empty(_out_shape(out_shape, M, K), dtype=torch.float16, device=dev)
    L = _lib.lib()
    drop = _drop_arg(dropout)
    with _device_ctx(dev):
        wp, wn = _gemm_scratch(L, dev, 0, M, K, N)
        rc = L.q4_gemm_bwd_dx_f16(dy2.data_ptr(), qweight.data_ptr(), qzeros.data_ptr(), scales.data_ptr(),
                                  gp, gs, _ptr(dyb), _ptr(lora_a), sr, sc, f32, float(lora_scale), R,
                                  out.data_ptr(), M, K, N, G, _drop_ref(drop), wp, wn, _stream(dev))
    _lib.check(rc, "q4_gemm_bwd_dx_f16")
    return out


LORA_GRAD_RANKS = tuple(range(2, 33, 2))


def lora_down(inp, w, dropout=None):
    """out fp16 [M, R] = inp fp16 [M, C] @ w^T for an adapter matrix view w [R, C] (fp16/fp32, any positive
    strides): xa = x @ A^T with w = lora_A.weight, dyb = dy @ B with w = lora_B.weight.t()  (models.py:66).
    dropout=(seed, p): out = dropout(inp) @ w^T with the counter-based mask of (seed, p)."""
    if _host is not None:
        return _host.lora_down(inp, w, None if dropout is None else (int(dropout[0]), float(dropout[1])))
    _require(inp.is_cuda and inp.dtype == torch.float16 and inp.dim() == 2 and inp.is_contiguous(),
             "inp must be a contiguous float16 [M, C] CUDA tensor")
    M, C = inp.shape
    _require(w.dim() == 2 and w.shape[1] == C and w.device == inp.device, "w must be an [R, C] view on the same device")
    R = w.shape[0]
    if M == 0:
        return torch.empty((0, R), dtype=torch.float16, device=inp.device)
    _require(1 <= R <= 64 and C % 32 == 0, "lora_down needs 1 <= R <= 64 and C % 32 == 0")
    f32 = _adapter_dtype_flag(w, "w")
    sr, sc = w.stride()
    _require(sr >= 1 and sc >= 1, "w must have positive strides")
    out = torch.empty((M, R), dtype=torch.float16, device=inp.device)
    drop = _drop_arg(dropout)
    with _device_ctx(inp.device):
        rc = _lib.lib().q4_lora_down_f16(inp.data_ptr(), w.data_ptr(), int(sr), int(sc), f32, out.data_ptr(),
                                         M, C, R, _drop_ref(drop), _stream(inp.device))
    _lib.check(rc, "q4_lora_down_f16")
    return out


def lora_grad(p, inp, alpha, transposed=False, dropout=None):
    """alpha * p^T @ inp in fp32 for p fp16 [M, R], inp fp16 [M, C], R in LORA_GRAD_RANKS.  Returns [R, C], or
    with transposed=True the same values stored as a contiguous [C, R] tensor (lora_B.weight's layout).
    dropout=(seed, p): inp is replaced by dropout(inp)."""
    _require(p.is_cuda and p.dtype == torch.float16 and p.dim() == 2 and p.is_contiguous(),
             "p must be a contiguous float16 [M, R] CUDA tensor")
    _require(inp.dtype == torch.float16 and inp.dim() == 2 and inp.is_contiguous() and inp.device == p.device
             and inp.shape[0] == p.shape[0], "inp must be a contiguous float16 [M, C] tensor on the same device")
    M, R = p.shape
    C = inp.shape[1]
    _require(R in LORA_GRAD_RANKS and C % 8 == 0, "lora_grad needs an even R in 2..32 and C % 8 == 0")
    dev = p.device
    if M == 0:                                               # empty batch: the gradient is zero
        return torch.zeros((C, R) if transposed else (R, C), dtype=torch.float32, device=dev)
    if transposed:
        out = torch.empty((C, R), dtype=torch.float32, device=dev)
        sr, sc = 1, R
    else:
        out = torch.empty((R, C), dtype=torch.float32, device=dev)
        sr, sc = C, 1
    L = _lib.lib()
    nbytes = L.q4_lora_grad_workspace_bytes(M, C, R)
    drop = _drop_arg(dropout)
    with _device_ctx(dev):
        ws = _scratch(dev, nbytes)
        rc = L.q4_lora_grad_f32(p.data_ptr(), inp.data_ptr(), out.data_ptr(), sr, sc, float(alpha), M, C, R,
                                _drop_ref(drop), ws.data_ptr(), ws.numel(), _stream(dev))
    _lib.check(rc, "q4_lora_grad_f32")
    return out


def lora_grad_pair(p1, inp1, p2, inp2, alpha, dropout=None, outs=None):
    """Both adapter gradients of a layer in one launch: returns (alpha * p1^T @ inp1 as [R, C1],
    alpha * p2^T @ inp2 stored as a contiguous [C2, R] tensor) -- dA from (dyb, x) and dB in lora_B.weight's
    layout from (xa, dy).  Same requirements as lora_grad; p1 and p2 share their shape.
    dropout=(seed, p): inp1 is replaced by dropout(inp1) (inp2 is left as it is)."""
    if _host is not None and outs is None:
        return _host.lora_grad_pair(p1, inp1, p2, inp2, float(alpha),
                                    None if dropout is None else (int(dropout[0]), float(dropout[1])))
    for p, inp in ((p1, inp1), (p2, inp2)):
        _require(p.is_cuda and p.dtype == torch.float16 and p.dim() == 2 and p.is_contiguous(),
                 "p must be a contiguous float16 [M, R] CUDA tensor")
        _require(inp.dtype == torch.float16 and inp.dim() == 2 and inp.is_contiguous() and inp.device == p.device
                 and inp.shape[0] == p.shape[0], "inp must be a contiguous float16 [M, C] tensor on the same device")
    _require(p1.shape == p2.shape and p1.device == p2.device, "the two rank-R operands must share shape and device")
    M, R = p1.shape
    C1, C2 = inp1.shape[1], inp2.shape[1]
    _require(R in LORA_GRAD_RANKS and C1 % 8 == 0 and C2 % 8 == 0, "lora_grad needs an even R in 2..32 and C % 8 == 0")
    dev = p1.device
    if M == 0:
        return (torch.zeros((R, C1), dtype=torch.float32, device=dev), torch.zeros((C2, R), dtype=torch.float32, device=dev))
    if outs is None:
        out1 = torch.empty((R, C1), dtype=torch.float32, device=dev)
        out2 = torch.empty((C2, R), dtype=torch.float32, device=dev)
    else:                                     # allocated by the caller (e.g. on another stream than the launch)
        out1, out2 = outs
        _require(out1.dtype == torch.float32 and tuple(out1.shape) == (R, C1) and out1.is_contiguous()
                 and out2.dtype == torch.float32 and tuple(out2.shape) == (C2, R) and out2.is_contiguous()
                 and out1.device == dev and out2.device == dev, "outs must be float32 [R, C1] and [C2, R] on the same device")
    L = _lib.lib()
    nbytes = L.q4_lora_grad_workspace_bytes(M, C1, R) + L.q4_lora_grad_workspace_bytes(M, C2, R)
    drop = _drop_arg(dropout)
    with _device_ctx(dev):
        ws = _scratch(dev, nbytes)
        rc = L.q4_lora_grad_pair_f32(p1.data_ptr(), inp1.data_ptr(), out1.data_ptr(), C1, 1, C1,
                                     p2.data_ptr(), inp2.data_ptr(), out2.data_ptr(), 1, R, C2,
                                     float(alpha), M, R, _drop_ref(drop), ws.data_ptr(), ws.numel(), _stream(dev))
    _lib.check(rc, "q4_lora_grad_pair_f32")
    return out1, out2


# ------------------------------------------------- quant_cuda-compatible entry points
def _infer_groupsize(K, G):
    return -(-K // G)


def _scales_half(scales):
    # the reference hands fp32 copies of fp16 scales to some kernels (matmul_utils_4bit.py:78,87)
    return scales if scales.dtype == torch.float16 else scales.half()


def vecquant4recons_v1(mat, res, scales, zeros):
    """quant_cuda.vecquant4recons_v1(mat, res, scales, zeros) -> None; res[K,N] = W of a v1 layer
    (quant_cuda.cpp:129-135)."""
    if res.dtype == torch.float16 and res.is_contiguous():
        dequant_v1(mat, scales, zeros, out=res)
    else:
        res.copy_(dequant_v1(mat, scales, zeros))


def vecquant2recons_v2(mat, res, scales, zeros, g_idx):
    """quant_cuda.vecquant2recons_v2(mat, res, scales, zeros, g_idx) -> None (quant_cuda.cpp:156-161)."""
    gs = _infer_groupsize(mat.shape[0] * 16, scales.shape[0])
    if res.dtype == torch.float16 and res.is_contiguous():
        dequant2(mat, zeros, _scales_half(scales), g_idx, gs, out=res)
    else:
        res.copy_(dequant2(mat, zeros, _scales_half(scales), g_idx, gs))


def vecquant4recons_v2(mat, res, scales, zeros, g_idx):
    """quant_cuda.vecquant4recons_v2(mat, res, scales, zeros, g_idx) -> None; res[K,N] = W.
    (quant_cuda.cpp:143-148).  fp16 scales: fp16 `res` is written in place, other dtypes via one cast.
    fp32 scales: the float kernel, `res` float32."""
    K = mat.shape[0] * 8
    gs = _infer_groupsize(K, scales.shape[0])
    _require(scales.dtype in (torch.float16, torch.float32),
             "scales must be float16 or float32 (the reference's float64 instantiation has no counterpart here)")
    if scales.dtype == torch.float32:
        # the reference dispatches on scales.type() (quant_cuda_kernel.cu:1173) and reads `res` as that type
        _require(res.dtype == torch.float32, "res must be float32 when scales are float32")
        if res.is_contiguous():
            dequant_f32(mat, zeros, scales, g_idx, gs, out=res)
        else:
            res.copy_(dequant_f32(mat, zeros, scales, g_idx, gs))
    elif res.dtype == torch.float16 and res.is_contiguous():
        dequant(mat, zeros, _scales_half(scales), g_idx, gs, out=res)
    else:
        res.copy_(dequant(mat, zeros, _scales_half(scales), g_idx, gs))


def _matmul_into(vec, mat, mul, scales, zeros, g_idx, groupsize):
    y = gemv(vec, mat, zeros, _scales_half(scales), g_idx, groupsize)
    mul.add_(y.to(mul.dtype))          # the reference kernels accumulate into a pre-zeroed `mul`


def vecquant4matmul(vec, mat, mul, scales, zeros, g_idx):
    """quant_cuda.vecquant4matmul (quant_cuda.cpp:55-61): mul += vec @ W, rows grouped by g_idx."""
    K = mat.shape[0] * 8
    _matmul_into(vec, mat, mul, scales, zeros, g_idx, _infer_groupsize(K, scales.shape[0]))


def vecquant4matmul_faster(vec, mat, mul, scales, zeros, g_idx, vec_height):
    """quant_cuda.vecquant4matmul_faster (quant_cuda.cpp:93-101)."""
    K = mat.shape[0] * 8
    assert vec_height * 2 == K
    _matmul_into(vec, mat, mul, scales, zeros, g_idx, _infer_groupsize(K, scales.shape[0]))


def vecquant4matmul_old_faster(vec, mat, mul, scales, zeros, groupsize, vec_height):
    """quant_cuda.vecquant4matmul_old_faster (quant_cuda.cpp:105-113): sequential groups of
    `groupsize` rows, g_idx not consulted (quant_cuda_kernel.cu:1024)."""
    K = mat.shape[0] * 8
    assert vec_height * 2 == K
    if groupsize is None or groupsize <= 0:
        groupsize = _infer_groupsize(K, scales.shape[0])
    _matmul_into(vec, mat, mul, scales, zeros, None, groupsize)


def vecquant4matmul_v1_faster(vec, mat, mul, scales, zeros):
    """quant_cuda.vecquant4matmul_v1_faster (quant_cuda.cpp:163-175): mul += vec @ W for a v1 layer."""
    mul.add_(gemv_v1(vec, mat, scales, zeros).to(mul.dtype))


def _unsupported(name):
    def fn(*args, **kwargs):
        raise NotImplementedError(f"{name}: not built for gfx950 (4-bit v2 runs fused; v1 and 2-bit v2 run through "
                                  "vecquant4recons_v1 / vecquant2recons_v2 + a dense GEMM, v1 decode through "
                                  "vecquant4matmul_v1_faster)")
    fn.__name__ = name
    return fn


for _n in ("vecquant2matmul", "vecquant3matmul", "vecquant8matmul", "vecquant2matmul_faster", "vecquant3matmul_faster",
           "vecquant4matmul_seq_v2", "vecquant4matmul_g"):
    globals()[_n] = _unsupported(_n)
