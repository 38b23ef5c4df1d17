"""ctypes binding of libq4gptq.so (C ABI declared in include/q4_gptq.h)."""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libq4gptq.so")
ABI_VERSION = 14

_lib = None

# name -> (restype, argtypes); must list every symbol of include/q4_gptq.h
_vp, _i, _sz, _f = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_float
SIGNATURES = {
    "q4_abi_version": (_i, []),
    "q4_error_string": (ctypes.c_char_p, [_i]),
    "q4_dequant_f16": (_i, [_vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _vp]),
    "q4_permute_rows": (_i, [_vp, _vp, _vp, _i, _i, _vp]),
    "q4_permute_cols_f16": (_i, [_vp, _vp, _vp, _i, _i, _vp]),
    "q4_gemv_workspace_bytes": (_sz, [_i, _i, _i]),
    "q4_gemv_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i, _i, _vp, _sz, _vp]),
    "q4_gemv_noalloc_max_outputs": (_sz, []),
    "q4_gemv_noalloc_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i, _i, _vp]),
    "q4_gemv_v1_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _sz, _vp]),
    "q4_gemv_sorted_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i, _i, _vp, _sz, _vp]),
    "q4_dequant_f32": (_i, [_vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _vp]),
    "q4_dequant_v1_f16": (_i, [_vp, _vp, _vp, _vp, _i, _i, _vp]),
    "q4_dequant2_f16": (_i, [_vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _vp]),
    "q4_gemm_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "q4_gemm_route": (_i, [_i, _i, _i, _i, _i, _i]),
    "q4_gemm_fwd_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _f, _i, _vp, _i, _i, _i, _i, _vp, _sz, _vp]),
    "q4_gemm_bwd_dx_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _f, _i, _vp, _i, _i, _i, _i, _vp, _vp, _sz, _vp]),
    "q4_lora_down_f16": (_i, [_vp, _vp, _i, _i, _i, _vp, _i, _i, _i, _vp, _vp]),
    "q4_lora_grad_workspace_bytes": (_sz, [_i, _i, _i]),
    "q4_lora_grad_f32": (_i, [_vp, _vp, _vp, _i, _i, _f, _i, _i, _i, _vp, _vp, _sz, _vp]),
    "q4_lora_grad_pair_f32": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp, _vp, _vp, _i, _i, _i, _f, _i, _i, _vp, _vp, _sz, _vp]),
    "q4_dropout_scale": (_f, [_f]),
    "q4_dropout_keep_u8": (_i, [_vp, _i, _i, _vp, _vp]),
}


class Dropout(ctypes.Structure):
    """q4_dropout_t of include/q4_gptq.h."""
    _fields_ = [("seed_lo", ctypes.c_uint32), ("seed_hi", ctypes.c_uint32), ("p", _f)]


class GemvLayer(ctypes.Structure):
    """q4_gemv_layer_t of include/q4_gptq.h."""
    _fields_ = [("x", _vp), ("qweight", _vp), ("qzeros", _vp), ("scales", _vp), ("y", _vp), ("N", _i)]


class Layer(ctypes.Structure):
    """q4_layer_t of include/q4_gptq.h."""
    _fields_ = [("qweight", _vp), ("qzeros", _vp), ("scales", _vp)]


SIGNATURES["q4_mlp_decode_workspace_bytes"] = (_sz, [_i, _i, _i])
SIGNATURES["q4_mlp_decode_status_offset"] = (_sz, [_i, _i, _i])
SIGNATURES["q4_mlp_decode_f16"] = (_i, [_vp, ctypes.POINTER(Layer), ctypes.POINTER(Layer), ctypes.POINTER(Layer), _i, _vp, _vp, _vp,
                                        _i, _i, _i, _vp, _sz, _vp])
class GemmLayer(ctypes.Structure):
    """q4_gemm_layer_t of include/q4_gptq.h."""
    _fields_ = [("act", _vp), ("qweight", _vp), ("qzeros", _vp), ("scales", _vp), ("bias", _vp), ("la", _vp), ("lb", _vp),
                ("lb_r", _i), ("lb_c", _i), ("lb_is_f32", _i), ("lb_scale", _f), ("R", _i), ("out", _vp), ("N", _i),
                ("drop", ctypes.POINTER(Dropout))]


SIGNATURES["q4_gemm_grouped_applicable"] = (_i, [_i, _i, _i, _i, ctypes.POINTER(_i)])
SIGNATURES["q4_gemm_grouped_workspace_bytes"] = (_sz, [_i, _i, _i, _i, ctypes.POINTER(_i)])
SIGNATURES["q4_gemm_grouped_fwd_f16"] = (_i, [ctypes.POINTER(GemmLayer), _i, _i, _i, _i, _vp])
SIGNATURES["q4_gemm_grouped_bwd_dx_f16"] = (_i, [ctypes.POINTER(GemmLayer), _i, _i, _vp, _i, _i, _vp, _sz, _vp])
MAX_GEMV_GROUP = 4
SIGNATURES["q4_gemv_grouped_workspace_bytes"] = (_sz, [_i, _i])
SIGNATURES["q4_gemv_grouped_f16"] = (_i, [ctypes.POINTER(GemvLayer), _i, _i, _i, _i, _i, _vp, _sz, _vp])


class Q4Error(RuntimeError):
    pass


def lib() -> ctypes.CDLL:
    """Load the HIP library; raise ImportError (never fall back) when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} not found: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "(hipcc --offload-arch=gfx950). There is no CPU fallback for the 4-bit kernels.")
    L = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    if L.q4_abi_version() != ABI_VERSION:
        raise ImportError(f"{LIB_PATH}: ABI version {L.q4_abi_version()} != expected {ABI_VERSION}; rebuild")
    _lib = L
    return L


def check(code: int, what: str) -> None:
    if code != 0:
        raise Q4Error(f"{what}: {lib().q4_error_string(code).decode()} (code {code})")
