"""No-GPU checks of the boundary: the C-ABI library loads and exports exactly what
include/q4_gptq.h declares, argument validation works without touching a device, and the
Python mirror keeps the reference's names, signatures, buffer layout and error types."""
import ctypes
import inspect
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "q4_gptq.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(q4_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from alpaca_lora_4bit_amd import _lib
    L = _lib.lib()
    names = _declared_functions()
    assert {"q4_dequant_f16", "q4_gemv_f16", "q4_gemm_fwd_f16", "q4_gemm_bwd_dx_f16",
            "q4_gemv_workspace_bytes", "q4_error_string", "q4_abi_version"} <= set(names)
    for n in names:
        assert hasattr(L, n), f"{n} declared in q4_gptq.h but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert sorted(_lib.SIGNATURES) == names
    assert L.q4_abi_version() == _lib.ABI_VERSION


def test_library_exports_nothing_but_the_declared_symbols():
    """The dynamic symbol table of the library holds exactly the functions of the header: internal launchers,
    planners and kernel stubs have hidden visibility."""
    import subprocess
    from alpaca_lora_4bit_amd import _lib
    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], check=True, capture_output=True, text=True).stdout
    exported = sorted(line.split()[-1] for line in out.splitlines() if len(line.split()) >= 3)
    assert exported == _declared_functions(), sorted(set(exported) ^ set(_declared_functions()))


def test_error_codes_and_validation_need_no_gpu():
    """Every entry point validates before launching: bad arguments return a code, never crash."""
    from alpaca_lora_4bit_amd import _lib
    L = _lib.lib()
    assert L.q4_error_string(0) == b"ok"
    for code in (-1, -2, -3, -4, -5, -6, -7):
        assert L.q4_error_string(code) not in (b"ok", b"unknown error")
    assert L.q4_error_string(-99) == b"unknown error"
    # null pointers
    assert L.q4_dequant_f16(None, None, None, None, 128, None, 256, 128, 2, None) == -1
    fake = ctypes.c_void_p(0x1000)           # aligned, never dereferenced: shape checks come first
    assert L.q4_dequant_f16(fake, fake, fake, None, 128, fake, 250, 128, 2, None) == -2      # K % 32
    assert L.q4_dequant_f16(fake, fake, fake, None, 128, fake, 256, 100, 2, None) == -2      # N % 64
    assert L.q4_dequant_f16(fake, fake, fake, None, 100, fake, 256, 128, 2, None) == -2      # groupsize % 32
    assert L.q4_dequant_f16(fake, fake, fake, None, 128, fake, 512, 128, 2, None) == -2      # G*groupsize < K
    odd = ctypes.c_void_p(0x1004)
    assert L.q4_dequant_f16(odd, fake, fake, None, 128, fake, 256, 128, 2, None) == -5
    assert L.q4_gemv_f16(fake, fake, fake, fake, None, 128, fake, 0, 17, 256, 128, 2, fake, 1 << 20, None) == -2
    assert L.q4_gemv_f16(fake, fake, fake, fake, None, 128, fake, 0, 1, 256, 128, 2, None, 0, None) == -3
    assert L.q4_gemv_f16(fake, fake, fake, fake, None, 128, fake, 0, 1, 256, 128, 2, fake, 8, None) == -3
    assert L.q4_gemv_sorted_f16(fake, fake, fake, fake, None, 128, fake, 0, 1, 256, 128, 2, fake, 1 << 20, None) == -1   # no perm
    assert L.q4_gemv_sorted_f16(fake, fake, fake, fake, fake, 128, fake, 0, 5, 256, 128, 2, fake, 1 << 20, None) == -2   # M > 4
    assert L.q4_gemv_sorted_f16(fake, fake, fake, fake, fake, 128, fake, 0, 4, 2048, 128, 16, None, 0, None) == -3
    assert L.q4_gemv_sorted_f16(fake, fake, fake, fake, fake, 128, fake, 0, 1, 512, 128, 4, fake, 1 << 20, None) == -2   # K < 1024
    assert L.q4_gemv_sorted_f16(fake, fake, fake, fake, fake, 128, fake, 0, 4, 8192, 128, 64, fake, 1 << 20, None) == -2  # rows do not fit in LDS
    assert L.q4_gemm_fwd_f16(fake, fake, fake, fake, None, 128, None, None, None, 0, 0, 0, 1.0, 0, fake, 64, 192, 128, 2, None, 0, None) == -2
    assert L.q4_gemm_fwd_f16(fake, fake, fake, fake, None, 128, None, fake, None, 1, 8, 0, 1.0, 8, fake, 64, 256, 128, 2, None, 0, None) == -1
    assert L.q4_gemm_fwd_f16(fake, fake, fake, fake, None, 128, None, fake, fake, 1, 12, 0, 1.0, 12, fake, 64, 256, 128, 2, None, 0, None) == -2
    assert L.q4_gemm_fwd_f16(fake, fake, fake, fake, None, 128, None, fake, fake, 0, 8, 1, 1.0, 8, fake, 64, 256, 128, 2, None, 0, None) == -2
    assert L.q4_gemm_bwd_dx_f16(fake, fake, fake, fake, None, 32, None, None, 0, 0, 0, 1.0, 0, fake, 64, 256, 128, 8, None, None, 0, None) == -2
    assert L.q4_gemm_fwd_f16(fake, fake, fake, fake, None, 128, None, None, None, 0, 0, 0, 1.0, 0, fake, 64, 256, 128, 2, ctypes.c_void_p(0x1010), 1 << 20, None) == -5
    assert L.q4_gemm_workspace_bytes(1, 2048, 4096, 4096) == 0            # enough tiles: no split
    assert L.q4_gemm_workspace_bytes(1, 64, 4096, 4096) == 8 * 64 * 4096 * 4    # 32 tiles -> 8 splits of fp32 partials
    assert L.q4_gemm_workspace_bytes(0, 64, 4096, 11008) == 8 * 64 * 4096 * 4
    # older layouts (dense dequantization only)
    assert L.q4_dequant_v1_f16(fake, fake, None, fake, 256, 128, None) == -1
    assert L.q4_gemv_v1_f16(fake, fake, fake, None, fake, 0, 1, 256, 128, fake, 1 << 20, None) == -1
    assert L.q4_gemv_v1_f16(fake, fake, fake, fake, fake, 0, 17, 256, 128, fake, 1 << 20, None) == -2
    assert L.q4_gemv_v1_f16(fake, fake, fake, fake, fake, 0, 1, 250, 128, fake, 1 << 20, None) == -2
    assert L.q4_gemv_v1_f16(fake, fake, fake, fake, fake, 0, 1, 256, 128, None, 0, None) == -3
    assert L.q4_gemv_v1_f16(fake, fake, fake, ctypes.c_void_p(0x1004), fake, 0, 1, 256, 128, fake, 1 << 20, None) == -5
    assert L.q4_dequant_v1_f16(fake, fake, fake, fake, 250, 128, None) == -2
    assert L.q4_dequant2_f16(fake, fake, fake, None, 128, fake, 264, 128, 3, None) == -2     # K % 16
    assert L.q4_dequant2_f16(fake, fake, fake, None, 128, odd, 256, 128, 2, None) == -5
    # adapter helpers
    assert L.q4_lora_down_f16(fake, None, 4096, 1, 1, fake, 64, 4096, 8, None, None) == -1
    assert L.q4_lora_down_f16(fake, fake, 4096, 1, 1, fake, 64, 4100, 8, None, None) == -2        # C % 32
    assert L.q4_lora_down_f16(fake, fake, 4096, 1, 1, fake, 64, 4096, 65, None, None) == -2       # R > 64
    assert L.q4_lora_down_f16(fake, ctypes.c_void_p(0x1002), 4096, 1, 1, fake, 64, 4096, 8, None, None) == -5
    assert L.q4_lora_grad_workspace_bytes(64, 4096, 8) == 0            # one row block: no partial sums
    assert L.q4_lora_grad_workspace_bytes(2048, 4096, 8) == 8 * 32 * 8 * 128 * 4      # 8 row blocks x 32 strips of [R, 128] fp32
    assert L.q4_lora_grad_workspace_bytes(2048, 4096, 12) == 8 * 32 * 12 * 128 * 4
    assert L.q4_lora_grad_workspace_bytes(2048, 4096, 7) == 0 and L.q4_lora_grad_workspace_bytes(2048, 4096, 34) == 0
    assert L.q4_lora_grad_f32(fake, fake, fake, 4096, 1, 1.0, 64, 4096, 7, None, fake, 1 << 20, None) == -2    # odd R
    assert L.q4_lora_grad_f32(fake, fake, fake, 4096, 1, 1.0, 64, 4096, 34, None, fake, 1 << 20, None) == -2   # R > 32
    assert L.q4_lora_grad_f32(fake, fake, fake, 4096, 1, 1.0, 2048, 4096, 8, None, None, 0, None) == -3
    assert L.q4_lora_grad_f32(fake, fake, fake, 4096, 1, 1.0, 2048, 4096, 8, None, fake, 1024, None) == -3
    assert L.q4_lora_grad_pair_f32(fake, fake, fake, 4096, 1, 4096, fake, fake, None, 1, 8, 4096, 1.0, 2048, 8, None, fake, 1 << 24, None) == -1
    assert L.q4_lora_grad_pair_f32(fake, fake, fake, 4096, 1, 4096, fake, fake, fake, 1, 8, 4100, 1.0, 2048, 8, None, fake, 1 << 24, None) == -2
    assert L.q4_lora_grad_pair_f32(fake, fake, fake, 4096, 1, 4096, fake, fake, fake, 1, 8, 4096, 1.0, 2048, 8, None, fake, 1 << 20, None) == -3  # needs 2 x 1 MiB
    # allocation-free GEMV: validated like q4_gemv_f16, plus the size of the built-in accumulator array
    assert L.q4_gemv_noalloc_max_outputs() == 16 * 32768
    assert L.q4_gemv_noalloc_f16(fake, fake, fake, fake, None, 128, fake, 0, 16, 256, 32832, 2, None) == -6
    assert L.q4_gemv_noalloc_f16(fake, fake, fake, fake, None, 128, fake, 0, 17, 256, 128, 2, None) == -2
    assert L.q4_gemv_noalloc_f16(None, fake, fake, fake, None, 128, fake, 0, 1, 256, 128, 2, None) == -1
    assert L.q4_gemv_noalloc_f16(fake, fake, fake, fake, None, 128, odd, 0, 1, 256, 128, 2, None) == -5
    # grouped GEMV: descriptors in host memory, validated layer by layer
    lay = (_lib.GemvLayer * 2)()
    for d in lay:
        d.x = d.qweight = d.qzeros = d.scales = d.y = 0x1000
        d.N = 128
    assert L.q4_gemv_grouped_workspace_bytes(4, 22016) == 4 * 22016 * 8
    assert L.q4_gemv_grouped_f16(None, 2, 128, 0, 1, 256, fake, 1 << 20, None) == -1
    assert L.q4_gemv_grouped_f16(lay, 5, 128, 0, 1, 256, fake, 1 << 20, None) == -2          # more than 4 layers
    assert L.q4_gemv_grouped_f16(lay, 2, 100, 0, 1, 256, fake, 1 << 20, None) == -2          # groupsize % 32
    assert L.q4_gemv_grouped_f16(lay, 2, 128, 0, 17, 256, fake, 1 << 20, None) == -2         # rows
    assert L.q4_gemv_grouped_f16(lay, 2, 128, 0, 1, 256, fake, 2047, None) == -3             # needs 2 * 128 * 8 bytes
    lay[1].N = 100
    assert L.q4_gemv_grouped_f16(lay, 2, 128, 0, 1, 256, fake, 1 << 20, None) == -2          # N % 64 of the second layer
    lay[1].N = 128
    lay[1].y = 0
    assert L.q4_gemv_grouped_f16(lay, 2, 128, 0, 1, 256, fake, 1 << 20, None) == -1
    # dropout descriptor: p outside [0, 1) is rejected, the realized scale is 32768 / (32768 - round(p * 32768))
    bad = _lib.Dropout(1, 2, 1.0)
    assert L.q4_lora_down_f16(fake, fake, 4096, 1, 1, fake, 64, 4096, 8, ctypes.byref(bad), None) == -2
    assert L.q4_dropout_keep_u8(fake, 4, 7, ctypes.byref(_lib.Dropout(1, 2, 0.5)), None) == -2       # C must be even
    assert L.q4_dropout_keep_u8(None, 4, 8, ctypes.byref(_lib.Dropout(1, 2, 0.5)), None) == -1
    assert abs(L.q4_dropout_scale(0.05) - 32768.0 / (32768 - 1638)) < 1e-6 and L.q4_dropout_scale(0.0) == 1.0
    assert L.q4_dropout_scale(1.5) == 0.0
    assert L.q4_gemv_workspace_bytes(16, 4096, 11008) == 16 * 11008 * 8
    assert L.q4_gemv_workspace_bytes(0, 4096, 11008) == 0


def test_streaming_kernel_selection_rules_need_no_gpu():
    """Which products of some hundred rows take the whole-reduction streaming kernels (host logic only): outputs that
    one round of at most 256 workgroups covers with row blocks of 32, 48 or 64 rows (grad-input: 32 or 48), sequential
    groups of a multiple of 128 rows, no act-order; the grad-input form only while the reduction is at most twice the
    output width; very long reductions only with the smallest row block."""
    from alpaca_lora_4bit_amd import _lib
    L = _lib.lib()
    def fwd(*a):
        return L.q4_gemm_route(1, *a) == 2            # Q4_ROUTE_STREAM

    def dx(*a):
        return L.q4_gemm_route(0, *a) == 2
    # (M, K, N, groupsize, has_gidx)
    assert fwd(128, 4096, 4096, 128, 0) and fwd(256, 4096, 4096, 128, 0) and fwd(65, 4096, 4096, 128, 0)
    assert not fwd(64, 4096, 4096, 128, 0)            # up to 64 rows and fewer than 128 strips: the other streaming kernel
    assert fwd(17, 4096, 11008, 128, 0) and fwd(64, 5120, 13824, 128, 0) and not fwd(16, 4096, 11008, 128, 0)
    assert not fwd(40, 4096, 16512, 128, 0)           # 258 strips
    assert not fwd(257, 4096, 4096, 128, 0)           # 64 strips x 5 blocks of 64 rows
    assert not fwd(128, 4096, 11008, 128, 0)          # 172 strips never fit one round above 64 rows
    assert fwd(192, 11008, 4096, 128, 0) and fwd(512, 2048, 2048, 128, 0) and not fwd(513, 2048, 2048, 128, 0)
    assert not fwd(128, 4096, 4096, 128, 1) and not fwd(128, 4096, 4096, 64, 0) and not fwd(128, 4096 + 64, 4096, 128, 0)
    assert fwd(65, 13824, 5120, 128, 0) and not fwd(128, 13824, 5120, 128, 0)     # long reduction: 32-row blocks only
    assert dx(49, 4096, 4096, 128, 0) and dx(256, 4096, 4096, 128, 0) and dx(384, 4096, 4096, 128, 0)
    assert not dx(48, 4096, 4096, 128, 0) and not dx(385, 4096, 4096, 128, 0)     # 32 blocks x 9 blocks of 48 rows
    assert dx(96, 11008, 4096, 128, 0) and not dx(97, 11008, 4096, 128, 0)        # 86 blocks x 2 / x 3
    assert not dx(128, 4096, 11008, 128, 0)           # reduction over 11008 columns for 4096 outputs
    assert not dx(128, 4096, 4096, 128, 1) and not dx(128, 4096, 4096, 64, 0)
    assert not fwd(128, 131072, 4096, 128, 0) and not dx(128, 4096, 131072, 128, 0)   # beyond the 32-bit offsets


def test_compiled_host_binding_is_built_and_matches_the_library():
    """The pybind11 host module (csrc/host/q4_host.cpp) sits next to the library, was built against the same ABI
    version, and quant_hip routes its operators through it.  Its argument checks run without a GPU."""
    import torch
    from alpaca_lora_4bit_amd import _lib, quant_hip
    host = quant_hip._host
    assert host is not None and host.abi_version() == _lib.ABI_VERSION
    for name in ("dequant", "gemv", "gemv_grouped", "gemm_fwd", "gemm_bwd_dx", "lora_down", "lora_grad_pair",
                 "reset_workspaces", "workspaces_are_zero"):
        assert callable(getattr(host, name))
    qw = torch.zeros((32, 128), dtype=torch.int32)
    qz = torch.zeros((2, 16), dtype=torch.int32)
    sc = torch.zeros((2, 128), dtype=torch.float16)
    with pytest.raises(ValueError, match="GPU"):                      # CPU tensors are refused, nothing is computed on the host
        host.gemv(torch.zeros((1, 256), dtype=torch.float16), qw, qz, sc, None, 128)
    with pytest.raises(ValueError):
        host.lora_down(torch.zeros((4, 64), dtype=torch.float16), torch.zeros((8, 64)))


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from alpaca_lora_4bit_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(ImportError, match="no CPU fallback"):
        _lib.lib()


def test_product_package_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "alpaca_lora_4bit_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, f"{f} mentions the oracle"


# ------------------------------------------------------------------ reference API surface
def test_quant_linear_buffers_are_the_checkpoint_format():
    import torch
    from alpaca_lora_4bit_amd.autograd_4bit import Autograd4bitQuantLinear
    m = Autograd4bitQuantLinear(4096, 11008, groupsize=128)
    sd = m.state_dict()
    assert set(sd) == {"qweight", "qzeros", "scales", "g_idx", "bias"}
    assert sd["qweight"].shape == (512, 11008) and sd["qweight"].dtype == torch.int32
    assert sd["qzeros"].shape == (32, 1376) and sd["qzeros"].dtype == torch.int32
    assert sd["scales"].shape == (32, 11008)
    assert sd["g_idx"].dtype == torch.int32 and torch.equal(sd["g_idx"], (torch.arange(4096) // 128).int())
    assert sd["bias"].shape == (11008,) and not sd["bias"].any()
    assert (m.bits, m.maxq, m.groupsize, m.is_v1_model, m.disable_bias) == (4, 15, 128, False, False)
    assert Autograd4bitQuantLinear(256, 128).groupsize == 256          # groupsize=-1 -> in_features
    assert "Autograd4bitQuantLinear" in str(type(m))


def test_autograd_function_signature_and_backend_registry():
    from alpaca_lora_4bit_amd import autograd_4bit as a
    assert a.backend == "cuda" and a.AutogradMatmul4bit is a.AutogradMatmul4bitCuda
    fwd = inspect.signature(a.AutogradMatmul4bitCuda.forward)
    assert list(fwd.parameters)[1:] == ["x", "qweight", "scales", "zeros", "g_idx", "bits", "maxq"]
    assert a.is_gptq_backend_available() and not a.is_triton_backend_available()
    with pytest.raises(ValueError):
        a.switch_backend_to("triton")
    with pytest.raises(ValueError):
        a.switch_backend_to("nope")
    a.switch_backend_to("cuda")
    with pytest.raises(NotImplementedError):
        a.AutogradMatmul4bitNotImplemented.apply(None, None, None, None, None, 4, 15)


def test_unsupported_bitwidth_and_layouts_raise_like_the_reference():
    import torch
    from alpaca_lora_4bit_amd import matmul_utils_4bit as mm4b
    from alpaca_lora_4bit_amd.autograd_4bit import Autograd4bitQuantLinear
    m = Autograd4bitQuantLinear(256, 128, groupsize=128, bits=3)
    with pytest.raises(ValueError, match="Unsupported bitwidth"):
        m(torch.zeros(1, 256))
    with pytest.raises(ValueError, match="CUDA"):      # fp zeros = v1 layout: dispatched, then rejected as CPU tensors
        mm4b.matmul4bit(torch.zeros(1, 256), torch.zeros(32, 128, dtype=torch.int32), torch.zeros(128, 1),
                        torch.zeros(128, 1))
    with pytest.raises(AssertionError):                # K mismatch, matmul_utils_4bit.py:71
        mm4b._matmul4bit_v2(torch.zeros(1, 128), torch.zeros(32, 128, dtype=torch.int32), torch.zeros(2, 128),
                            torch.zeros(2, 16, dtype=torch.int32), torch.zeros(256, dtype=torch.int32))
    with pytest.raises(AssertionError):
        mm4b._matmul4bit_v2_recons(torch.zeros(32, 100), torch.zeros(32, 128, dtype=torch.int32), torch.zeros(2, 128),
                                   torch.zeros(2, 16, dtype=torch.int32), torch.zeros(256, dtype=torch.int32),
                                   transpose=True)


def test_module_knobs_exist_with_reference_names():
    from alpaca_lora_4bit_amd import matmul_utils_4bit as mm4b
    for name in ("buffer_mat_dic", "use_new", "auto_switch", "auto_switch_thd", "debug", "faster_mode",
                 "valid_faster_mode", "act_order", "cache_buffer", "get_buffer", "matmul4bit", "_matmul4bit_v2",
                 "_matmul4bit_v2_recons", "_matmul4bit_v1", "_matmul4bit_v1_recons", "_matmul2bit_v2_recons", "v2_to_v1"):
        assert hasattr(mm4b, name), name
    assert mm4b.faster_mode == "old_faster" and mm4b.act_order is False and mm4b.cache_buffer is True


def test_quant_cuda_mirror_exports_the_pybind_names():
    from alpaca_lora_4bit_amd import quant_hip
    for name in ("vecquant2matmul", "vecquant3matmul", "vecquant4matmul", "vecquant8matmul", "vecquant2matmul_faster",
                 "vecquant3matmul_faster", "vecquant4matmul_faster", "vecquant4matmul_old_faster",
                 "vecquant4matmul_v1_faster", "vecquant4recons_v1", "vecquant4recons_v2", "vecquant2recons_v2",
                 "vecquant4matmul_seq_v2", "vecquant4matmul_g"):
        assert callable(getattr(quant_hip, name)), name
    with pytest.raises(NotImplementedError):
        quant_hip.vecquant2matmul()
    assert list(inspect.signature(quant_hip.vecquant4matmul_v1_faster).parameters) == ["vec", "mat", "mul", "scales", "zeros"]
    assert list(inspect.signature(quant_hip.vecquant4recons_v1).parameters) == ["mat", "res", "scales", "zeros"]
    assert list(inspect.signature(quant_hip.vecquant2recons_v2).parameters) == ["mat", "res", "scales", "zeros", "g_idx"]
    assert list(inspect.signature(quant_hip.vecquant4recons_v2).parameters) == ["mat", "res", "scales", "zeros", "g_idx"]
    assert list(inspect.signature(quant_hip.vecquant4matmul_old_faster).parameters) == \
        ["vec", "mat", "mul", "scales", "zeros", "groupsize", "vec_height"]


def test_host_checks_reject_cpu_tensors_and_bad_dtypes():
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    qw = torch.zeros(32, 128, dtype=torch.int32)
    with pytest.raises(ValueError, match="GPU"):
        quant_hip.dequant(qw, torch.zeros(2, 16, dtype=torch.int32), torch.zeros(2, 128, dtype=torch.float16), None, 128)


def test_make_quant_and_find_layers_and_model_to_half():
    import torch
    import torch.nn as nn
    from alpaca_lora_4bit_amd import autograd_4bit as a

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.q_proj = nn.Linear(256, 256, bias=False)
            self.mlp = nn.Sequential(nn.Linear(256, 512, bias=False), nn.Linear(512, 256, bias=False))

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.layers = nn.ModuleList([Block(), Block()])
            self.lm_head = nn.Linear(256, 1000, bias=False)

    net = Net()
    layers = a.find_layers(net)
    assert set(layers) == {"layers.0.q_proj", "layers.0.mlp.0", "layers.0.mlp.1", "layers.1.q_proj", "layers.1.mlp.0",
                           "layers.1.mlp.1", "lm_head"}
    del layers["lm_head"]
    a.make_quant_for_4bit_autograd(net, layers, groupsize=128)
    assert isinstance(net.layers[0].q_proj, a.Autograd4bitQuantLinear) and isinstance(net.lm_head, nn.Linear)
    assert net.layers[1].mlp[0].qweight.shape == (32, 512)
    a.model_to_half(net)
    assert net.layers[0].q_proj.scales.dtype == torch.float16 and net.layers[0].q_proj.bias.dtype == torch.float16
    assert net.layers[0].q_proj.qweight.dtype == torch.int32


def test_linear4bitlt_and_injection_without_peft():
    import torch.nn as nn
    from alpaca_lora_4bit_amd import models
    from alpaca_lora_4bit_amd.autograd_4bit import Autograd4bitQuantLinear

    class Attn(nn.Module):
        def __init__(self):
            super().__init__()
            self.q_proj = Autograd4bitQuantLinear(256, 256, groupsize=128)
            self.k_proj = Autograd4bitQuantLinear(256, 256, groupsize=128)
            self.v_proj = Autograd4bitQuantLinear(256, 256, groupsize=128)

    net = nn.ModuleList([Attn(), Attn()])
    old_q = net[0].q_proj
    new = models.inject_lora_layers(net, ("q_proj", "v_proj"), r=8, lora_alpha=16)
    assert set(new) == {"0.q_proj", "0.v_proj", "1.q_proj", "1.v_proj"}
    lt = net[0].q_proj
    assert isinstance(lt, models.Linear4bitLt) and isinstance(lt, Autograd4bitQuantLinear) and "Linear4bitLt" in str(type(lt))
    assert lt.qweight is old_q.qweight and lt.scales is old_q.scales and lt.g_idx is old_q.g_idx     # shared, not copied
    assert lt.scaling["default"] == 2.0 and lt.lora_A["default"].weight.shape == (8, 256)
    assert lt.lora_B["default"].weight.shape == (256, 8) and not lt.lora_B["default"].weight.any()
    trainable = [n for n, p in net.named_parameters() if p.requires_grad]
    assert len(trainable) == 8 and all("lora_" in n for n in trainable)
    assert lt.weight.device == lt.qweight.device
    assert isinstance(net[0].k_proj, Autograd4bitQuantLinear) and not isinstance(net[0].k_proj, models.Linear4bitLt)


def test_alias_package_resolves_reference_import_paths():
    import alpaca_lora_4bit_amd as pkg
    pkg.install_as_alpaca_lora_4bit()
    from alpaca_lora_4bit import autograd_4bit  # noqa: F401
    import alpaca_lora_4bit.matmul_utils_4bit as mm4b
    from alpaca_lora_4bit.monkeypatch.peft_tuners_lora_monkey_patch import replace_peft_model_with_int4_lora_model
    from alpaca_lora_4bit import quant_cuda
    assert mm4b.quant_hip is quant_cuda and callable(replace_peft_model_with_int4_lora_model)
    try:
        import peft  # noqa: F401
    except ImportError:
        with pytest.raises(ImportError, match="peft"):
            replace_peft_model_with_int4_lora_model()


def test_amp_wrapper_interface():
    import torch
    from alpaca_lora_4bit_amd.amp_wrapper import AMPWrapper

    class M(torch.nn.Module):
        def forward(self, x):
            return torch.is_autocast_enabled("cpu"), x

        def generate(self, x):
            return torch.is_autocast_enabled("cpu")

    m = M()
    w = AMPWrapper(m, {"enabled": True, "device_type": "cpu", "dtype": torch.bfloat16})
    w.apply_forward()
    w.apply_generate()
    assert m.forward(1)[0] is True and m.generate(1) is True
    assert m.non_autocast_forward(1)[0] is False
    assert AMPWrapper(m).options == {"enabled": True, "device_type": "cuda"}


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "--gpus must be 1" in r.stderr
