"""Act-order layers: the one-time row sort (q4_permute_rows + gathered x) and the direct
gather kernels must both agree with the CPU oracle; the repack itself is bit-exact."""
import numpy as np
import pytest

from conftest import rel_err, to_cuda_layer

pytestmark = pytest.mark.gpu
TOL = 1e-2


@pytest.fixture(params=[True, False], ids=["repack", "gather"])
def repack(request):
    from alpaca_lora_4bit_amd import quant_hip
    old = quant_hip.actorder_repack
    quant_hip.actorder_repack = request.param
    yield request.param
    quant_hip.actorder_repack = old


def test_permute_rows_bit_exact(oracle):
    import torch
    from alpaca_lora_4bit_amd import _lib, quant_hip
    rng = np.random.default_rng(3)
    K, N = 512, 192
    codes = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    perm = rng.permutation(K).astype(np.int32)
    qw = torch.from_numpy(oracle.pack_qweight(codes)).cuda()
    out = torch.empty_like(qw)
    rc = _lib.lib().q4_permute_rows(qw.data_ptr(), torch.from_numpy(perm).cuda().data_ptr(), out.data_ptr(), K, N,
                                    torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    assert np.array_equal(out.cpu().numpy(), oracle.pack_qweight(codes[perm]))
    assert _lib.lib().q4_permute_rows(qw.data_ptr(), qw.data_ptr(), qw.data_ptr(), K, N, None) == -2   # in place refused


@pytest.mark.parametrize("M,K", [(1, 128), (7, 4096), (64, 4096), (300, 11008), (2049, 5120), (33, 32768), (1000, 256)])
def test_permute_cols_bit_exact(M, K):
    """q4_permute_cols_f16 through the C ABI: out[m, p] = in[m, idx[p]] for a permutation and for an index vector with
    repeats (1, 2, 5, 16 rows per workgroup and a last workgroup with fewer); argument checks."""
    import torch
    from alpaca_lora_4bit_amd import _lib, quant_hip
    g = torch.Generator().manual_seed(M + K)
    x = torch.randn((M, K), generator=g).half().cuda()
    L = _lib.lib()
    st = torch.cuda.current_stream().cuda_stream
    for idx in (torch.randperm(K, generator=g).int().cuda(), torch.randint(0, K, (K,), generator=g).int().cuda()):
        out = torch.full_like(x, float("nan"))
        assert L.q4_permute_cols_f16(x.data_ptr(), idx.data_ptr(), out.data_ptr(), M, K, st) == 0
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), x.index_select(1, idx.long()).view(torch.int16))
        assert torch.equal(quant_hip.permute_cols(x, idx).view(torch.int16), out.view(torch.int16))
    assert L.q4_permute_cols_f16(x.data_ptr(), idx.data_ptr(), x.data_ptr(), M, K, st) == -2          # in place refused
    assert L.q4_permute_cols_f16(x.data_ptr(), idx.data_ptr(), out.data_ptr(), M, K + 4, st) == -2      # K % 8
    assert L.q4_permute_cols_f16(x.data_ptr(), idx.data_ptr(), out.data_ptr(), M, 32768 + 8, st) == -2  # a row must fit the LDS
    assert L.q4_permute_cols_f16(None, idx.data_ptr(), out.data_ptr(), M, K, st) == -1
    assert L.q4_permute_cols_f16(x.data_ptr() + 2, idx.data_ptr(), out.data_ptr(), M, K, st) == -5


def test_sorted_layer_plan(oracle):
    """Sorted copy dequantizes (with sequential groups) to the row-permuted dense weight."""
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    layer = oracle.make_layer(1024, 256, 128, act_order=True, seed=12)
    t = to_cuda_layer(layer)
    plan = quant_hip.sorted_layer(t["qweight"], t["g_idx"], 8)
    assert plan is not None
    perm, inv, qs, gs = plan
    assert gs == 128 and torch.equal(perm.long()[inv.long()], torch.arange(1024, device="cuda"))
    assert torch.equal(t["g_idx"].long()[perm.long()], torch.arange(1024, device="cuda") // 128)
    W = oracle.dequant_v2(layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    Ws = quant_hip.dequant(qs, t["qzeros"], t["scales"], None, 128).cpu().numpy()
    assert np.array_equal(Ws.view(np.uint16), W[perm.cpu().numpy()].view(np.uint16))
    assert quant_hip.sorted_layer(t["qweight"], t["g_idx"], 8) is plan                # cached
    # groups of unequal size cannot be sorted into the sequential layout
    g2 = t["g_idx"].clone()
    g2[0] = (g2[0] + 1) % 8
    assert quant_hip.sorted_layer(t["qweight"], g2, 8) is None


@pytest.mark.parametrize("K,N,M", [(5120, 13824, 1), (5120, 13824, 16), (512, 256, 5), (5120, 13824, 4), (512, 256, 2),
                                   (1408, 256, 3), (256, 128, 1)])
def test_actorder_gemv(oracle, repack, K, N, M):
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    layer = oracle.make_layer(K, N, 128, act_order=True, seed=K + N)
    t = to_cuda_layer(layer)
    x = oracle.make_activations(M, K, seed=M)
    ref = oracle.matmul_recons(x, layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    y = quant_hip.gemv(torch.from_numpy(x).cuda(), t["qweight"], t["qzeros"], t["scales"], t["g_idx"], 128)
    assert rel_err(y.cpu().numpy(), ref) <= TOL


def test_sorted_gemv_gathers_activations_in_the_kernel(oracle):
    """Up to 4 rows: q4_gemv_sorted_f16 takes the original x and the permutation and gives the bits of the
    sequential kernel run on x gathered beforehand; it also accumulates into y and leaves the workspace zero."""
    import torch
    from alpaca_lora_4bit_amd import _lib, quant_hip
    K, N = 1408, 384                                      # 11 chunks of 128: the second workgroup of a strip is partly idle
    layer = oracle.make_layer(K, N, 128, act_order=True, seed=9)
    t = to_cuda_layer(layer)
    perm, _, qsorted, gs = quant_hip.sorted_layer(t["qweight"], t["g_idx"], K // 128)
    L = _lib.lib()
    for M in (1, 3, 4):
        x = torch.from_numpy(oracle.make_activations(M, K, seed=M)).cuda()
        want = quant_hip.gemv(x.index_select(1, perm.long()).contiguous(), qsorted, t["qzeros"], t["scales"], None, gs)
        got = quant_hip.gemv(x, t["qweight"], t["qzeros"], t["scales"], t["g_idx"], 128)
        assert torch.equal(got, want)
        base = torch.randn(M, N, device="cuda").half()
        acc = base.clone()
        quant_hip.gemv(x, t["qweight"], t["qzeros"], t["scales"], t["g_idx"], 128, out=acc, accumulate=True)
        assert torch.allclose(acc.float(), base.float() + want.float(), rtol=0, atol=2e-3 * float(want.abs().max()))
    ws = torch.zeros(L.q4_gemv_workspace_bytes(4, K, N), dtype=torch.uint8, device="cuda")
    y = torch.empty(4, N, dtype=torch.float16, device="cuda")
    x = torch.from_numpy(oracle.make_activations(4, K, seed=3)).cuda()
    rc = L.q4_gemv_sorted_f16(x.data_ptr(), qsorted.data_ptr(), t["qzeros"].data_ptr(), t["scales"].data_ptr(),
                              perm.data_ptr(), gs, y.data_ptr(), 0, 4, K, N, K // 128, ws.data_ptr(), ws.numel(), None)
    torch.cuda.synchronize()
    assert rc == 0 and int(ws.count_nonzero()) == 0


@pytest.mark.parametrize("K,N,M", [(5120, 13824, 512), (512, 384, 40)])
def test_actorder_gemm_forward_backward_lora(oracle, repack, K, N, M):
    """Config 3 (M=512) forward, plus backward-dx with the adapter term through the permutation."""
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    layer = oracle.make_layer(K, N, 128, act_order=True, seed=K + N + 7)
    t = to_cuda_layer(layer)
    A, B = oracle.make_lora(K, N, 8, seed=5)
    A16, B16 = A.astype(np.float16), B.astype(np.float16)
    x = oracle.make_activations(M, K, seed=1)
    dy = oracle.make_activations(M, N, seed=2)
    W = oracle.dequant_v2(layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"]).astype(np.float64)
    yref = oracle.lora_forward(x, W, A16, B16, 2.0)
    dxref, _, _ = oracle.lora_backward(x, dy, W, A16, B16, 2.0)
    xt, dyt = torch.from_numpy(x).cuda(), torch.from_numpy(dy).cuda()
    a16, b16 = torch.from_numpy(A16).cuda(), torch.from_numpy(B16).cuda()
    y = quant_hip.gemm_fwd(xt, t["qweight"], t["qzeros"], t["scales"], t["g_idx"], 128, xa=xt @ a16.t(),
                           lora_bt=b16.t(), lora_scale=2.0)
    dx = quant_hip.gemm_bwd_dx(dyt, t["qweight"], t["qzeros"], t["scales"], t["g_idx"], 128, dyb=dyt @ b16,
                               lora_a=a16, lora_scale=2.0)
    assert rel_err(y.cpu().numpy(), yref) <= TOL
    assert rel_err(dx.cpu().numpy(), dxref) <= TOL
