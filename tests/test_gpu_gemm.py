"""Fused dequant + MFMA GEMMs (forward, backward-dx, LoRA steps) vs the CPU oracle.
Tolerance: max|out - ref| <= 1e-2 * max|ref| against the fp32-accumulated reference."""
import numpy as np
import pytest

from conftest import rel_err, to_cuda_layer

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _t(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("K,N,gs,act", [(256, 128, 128, False), (256, 256, 64, False), (512, 384, 128, True),
                                        (4096, 4096, 128, False), (1024, 256, 1024, False),
                                        (1408, 256, 128, False), (1408, 256, 128, True)])   # 22 steps: uneven split-K
@pytest.mark.parametrize("M", [17, 128, 300])
def test_gemm_forward(oracle, K, N, gs, act, M):
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    layer = oracle.make_layer(K, N, gs, act_order=act, seed=K + N + 1)
    t = to_cuda_layer(layer)
    x = oracle.make_activations(M, K, seed=M)
    ref = oracle.matmul_recons(x, layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    y = quant_hip.gemm_fwd(_t(x), t["qweight"], t["qzeros"], t["scales"], t["g_idx"], gs)
    torch.cuda.synchronize()
    assert rel_err(y.cpu().numpy(), ref) <= TOL
    assert rel_err(y.cpu().numpy(), ref) <= 2e-3


@pytest.mark.parametrize("K,N,gs,act", [(256, 128, 128, False), (256, 256, 64, False), (512, 384, 128, True),
                                        (4096, 4096, 128, False), (256, 1408, 128, False)])   # reduction of 22 steps
@pytest.mark.parametrize("M", [17, 128, 300])
def test_gemm_backward_dx(oracle, K, N, gs, act, M):
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    layer = oracle.make_layer(K, N, gs, act_order=act, seed=K + N + 2)
    t = to_cuda_layer(layer)
    dy = oracle.make_activations(M, N, seed=M + 5)
    ref = oracle.matmul_recons_t(dy, layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    dx = quant_hip.gemm_bwd_dx(_t(dy), t["qweight"], t["qzeros"], t["scales"], t["g_idx"], gs)
    torch.cuda.synchronize()
    assert rel_err(dx.cpu().numpy(), ref) <= TOL
    assert rel_err(dx.cpu().numpy(), ref) <= 2e-3


@pytest.mark.parametrize("K,N,gs", [(4096, 11008, 128), (11008, 4096, 128), (4096, 4096, 256), (1408, 384, 256), (128, 128, 128)])
@pytest.mark.parametrize("M", [17, 24, 32, 33, 48])
def test_streaming_grad_input_17_to_48_rows(oracle, K, N, gs, M):
    """The weight-streaming grad-input kernel (17..48 rows, sequential groups of a multiple of 128 rows) against the
    float64 product of dy with the bit-exact dense W, and against the tiled kernel that takes 49 rows and more."""
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    layer = oracle.make_layer(K, N, gs, act_order=False, seed=K + N + M)
    t = to_cuda_layer(layer)
    dy = _t(oracle.make_activations(M, N, seed=M + 9))
    W = quant_hip.dequant(t["qweight"], t["qzeros"], t["scales"], t["g_idx"], gs)
    ref = dy.double() @ W.double().t()
    dx = quant_hip.gemm_bwd_dx(dy, t["qweight"], t["qzeros"], t["scales"], None, gs)
    assert dx.shape == (M, K)
    err = float((dx.double() - ref).abs().max() / ref.abs().max())
    assert err <= TOL and err <= 2e-3, err
    # a sample of rows against the CPU oracle itself (the line above rests on the library's own dense W)
    rows = [0, M // 2, M - 1]
    oref = oracle.matmul_recons_t(dy.cpu().numpy()[rows], layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    assert rel_err(dx.cpu().numpy()[rows], oref) <= 2e-3
    again = quant_hip.gemm_bwd_dx(dy, t["qweight"], t["qzeros"], t["scales"], None, gs)
    assert torch.equal(dx, again)                                   # ordered partial sums: bit-reproducible
    big = torch.cat([dy, torch.zeros(49 - M, N, dtype=dy.dtype, device=dy.device)])     # 49 rows: the tiled kernel
    tiled = quant_hip.gemm_bwd_dx(big, t["qweight"], t["qzeros"], t["scales"], None, gs)[:M]
    assert float((dx.float() - tiled.float()).abs().max() / ref.abs().max()) <= 2e-3


def test_gemm_equals_dense_matmul_of_dequantized_weight(oracle):
    """The fused kernels hold the same fp16 W in LDS that the dense dequant writes: against
    torch.matmul(x, W_hip) the only difference is fp32 summation order."""
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    layer = oracle.make_layer(1024, 512, 128, seed=77)
    t = to_cuda_layer(layer)
    W = quant_hip.dequant(t["qweight"], t["qzeros"], t["scales"], t["g_idx"], 128)
    x = _t(oracle.make_activations(256, 1024, seed=1))
    dy = _t(oracle.make_activations(256, 512, seed=2))
    y = quant_hip.gemm_fwd(x, t["qweight"], t["qzeros"], t["scales"], t["g_idx"], 128)
    dx = quant_hip.gemm_bwd_dx(dy, t["qweight"], t["qzeros"], t["scales"], t["g_idx"], 128)
    yr = (x.float() @ W.float())
    dxr = (dy.float() @ W.float().t())
    assert float((y.float() - yr).abs().max() / yr.abs().max()) <= 1e-3
    assert float((dx.float() - dxr).abs().max() / dxr.abs().max()) <= 1e-3


@pytest.mark.parametrize("act", [False, True])
@pytest.mark.parametrize("M,K,N,r", [(2048, 4096, 4096, 8), (130, 256, 384, 16), (64, 512, 128, 64),
                                     (1024, 4096, 4096, 8), (512, 11008, 4096, 16)])   # 256-row tiles, reduction split 2 / 4 ways
def test_gemm_lora_steps(oracle, M, K, N, r, act):
    """Config 2 shape (and small ones): forward with bias + adapter, backward-dx with adapter."""
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    layer = oracle.make_layer(K, N, 128, act_order=act, seed=31)
    t = to_cuda_layer(layer)
    A, B = oracle.make_lora(K, N, r, seed=31)
    scaling = 2.0
    x = oracle.make_activations(M, K, seed=41)
    dy = oracle.make_activations(M, N, seed=42)
    bias = (np.random.default_rng(1).standard_normal(N) * 0.1).astype(np.float16)
    W = oracle.dequant_v2(layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"]).astype(np.float64)
    A16, B16 = A.astype(np.float16), B.astype(np.float16)
    yref = oracle.lora_forward(x, W, A16, B16, scaling, bias=bias)
    dxref, _, _ = oracle.lora_backward(x, dy, W, A16, B16, scaling)

    xt, dyt = _t(x), _t(dy)
    a16, b16 = _t(A16), _t(B16)
    xa = xt @ a16.t()
    y = quant_hip.gemm_fwd(xt, t["qweight"], t["qzeros"], t["scales"], t["g_idx"], 128, bias=_t(bias),
                           xa=xa, lora_bt=b16.t(), lora_scale=scaling)          # strided view of B [N, r]
    dyb = dyt @ b16
    dx = quant_hip.gemm_bwd_dx(dyt, t["qweight"], t["qzeros"], t["scales"], t["g_idx"], 128, dyb=dyb, lora_a=a16,
                               lora_scale=scaling)
    # a contiguous [r, N] copy of the adapter matrix must give the same bits as the strided view
    y_c = quant_hip.gemm_fwd(xt, t["qweight"], t["qzeros"], t["scales"], t["g_idx"], 128, bias=_t(bias),
                             xa=xa, lora_bt=b16.t().contiguous(), lora_scale=scaling)
    assert torch.equal(y, y_c)
    torch.cuda.synchronize()
    assert rel_err(y.cpu().numpy(), yref) <= TOL
    assert rel_err(dx.cpu().numpy(), dxref) <= TOL
    # the adapter term must actually be there: without it the error is visible
    y0 = quant_hip.gemm_fwd(xt, t["qweight"], t["qzeros"], t["scales"], t["g_idx"], 128, bias=_t(bias))
    assert rel_err(y0.cpu().numpy(), yref) > rel_err(y.cpu().numpy(), yref)


@pytest.mark.parametrize("M,K,N,gs,act,r", [(9300, 1024, 1024, 128, False, 8), (9217, 1024, 1024, 128, True, 0),
                                            (9300, 1024, 1024, 64, False, 16), (2350, 4096, 4096, 128, False, 8),
                                            (2305, 512, 4096, 256, False, 0)])
def test_wide_tiles_256x256(oracle, M, K, N, gs, act, r):
    """Outputs with at least 144 tiles of 256 x 256 run the eight-wavefront wide tile (forward and grad-input, with
    bias, adapter step and the masked adapter term): against fp32 products with the bit-exact dense W on the GPU."""
    import torch
    from alpaca_lora_4bit_amd import _lib, quant_hip
    layer = oracle.make_layer(K, N, gs, act_order=act, seed=M + K)
    t = to_cuda_layer(layer)
    g = torch.Generator(device="cuda").manual_seed(M)
    x = torch.randn((M, K), device="cuda", generator=g).half()
    dy = torch.randn((M, N), device="cuda", generator=g).half()
    bias = (torch.randn(N, device="cuda", generator=g) * 0.1).half()
    W = quant_hip.dequant(t["qweight"], t["qzeros"], t["scales"], t["g_idx"], gs).float()
    gi = t["g_idx"] if (act or gs % 64) else None
    kw_f, kw_b = {}, {}
    yref = x.float() @ W + bias.float()
    dxref = dy.float() @ W.t()
    if r:
        A = (torch.randn((r, K), device="cuda", generator=g) * 0.05)          # fp32 adapter matrices, read in place
        B = (torch.randn((N, r), device="cuda", generator=g) * 0.05)
        xa = quant_hip.lora_down(x, A)
        dyb = quant_hip.lora_down(dy, B.t())
        kw_f = dict(xa=xa, lora_bt=B.t(), lora_scale=2.0)
        kw_b = dict(dyb=dyb, lora_a=A, lora_scale=2.0)
        yref = yref + 2.0 * (xa.float() @ B.half().float().t())
        dxref = dxref + 2.0 * (dyb.float() @ A.half().float())
    y = quant_hip.gemm_fwd(x, t["qweight"], t["qzeros"], t["scales"], gi, gs, bias=bias, **kw_f)
    dx = quant_hip.gemm_bwd_dx(dy, t["qweight"], t["qzeros"], t["scales"], gi, gs, **kw_b)
    assert y.shape == (M, N) and dx.shape == (M, K)
    for got, ref in ((y, yref), (dx, dxref)):
        err = float((got.float() - ref).abs().max() / ref.abs().max())
        assert err <= TOL and err <= 2e-3, err
    # a sample of rows from different row tiles against the CPU oracle itself (float64, oracle's own dense W)
    rows = np.array([0, 255, 256, 1000, M - 257, M - 1])
    xs, dys = x.cpu().numpy()[rows], dy.cpu().numpy()[rows]
    oy = oracle.matmul_recons(xs, layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"]) + bias.float().cpu().numpy()
    odx = oracle.matmul_recons_t(dys, layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    if r:
        oy = oy + 2.0 * (xa.float().cpu().numpy()[rows].astype(np.float64) @ B.half().float().cpu().numpy().astype(np.float64).T)
        odx = odx + 2.0 * (dyb.float().cpu().numpy()[rows].astype(np.float64) @ A.half().float().cpu().numpy().astype(np.float64))
    assert rel_err(y.cpu().numpy()[rows], oy) <= 2e-3 and rel_err(dx.cpu().numpy()[rows], odx) <= 2e-3
    # the forward product of every case has at least 144 wide tiles: it runs unsplit and wants no workspace
    assert (N // 256) * -(-M // 256) >= 144 and _lib.lib().q4_gemm_workspace_bytes(1, M, K, N) == 0
    if r:
        # masked adapter term of the grad-input (dropout in front of lora_A): only kept positions carry it
        drop = (1234, 0.25)
        keep = quant_hip.dropout_keep_mask(M, K, drop[0], drop[1], x.device).float()
        dxm = quant_hip.gemm_bwd_dx(dy, t["qweight"], t["qzeros"], t["scales"], gi, gs, dropout=drop, **kw_b)
        ref = dy.float() @ W.t() + keep * quant_hip.dropout_scale(drop[1]) * 2.0 * (dyb.float() @ A.half().float())
        assert float((dxm.float() - ref).abs().max() / ref.abs().max()) <= 2e-3


def test_gemm_rejects_unsupported_shapes(oracle):
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    layer = oracle.make_layer(192, 128, 64, seed=1)      # K % 128 != 0
    t = to_cuda_layer(layer)
    x = _t(oracle.make_activations(32, 192, seed=1))
    with pytest.raises(quant_hip.Q4Error):
        quant_hip.gemm_fwd(x, t["qweight"], t["qzeros"], t["scales"], t["g_idx"], 64)


def test_split_k_is_reproducible_and_matches_unsplit(oracle):
    """Few tiles: the reduction is split and the fp32 partial tiles are added in a fixed order."""
    import torch
    from alpaca_lora_4bit_amd import _lib, quant_hip
    K, N, M = 4096, 512, 40
    assert _lib.lib().q4_gemm_workspace_bytes(1, M, K, N) > 0            # this shape does get split
    layer = oracle.make_layer(K, N, 128, seed=77)
    t = to_cuda_layer(layer)
    x = torch.from_numpy(oracle.make_activations(M, K, seed=4)).cuda()
    bias = torch.randn(N, device="cuda").half()
    y1 = quant_hip.gemm_fwd(x, t["qweight"], t["qzeros"], t["scales"], None, 128, bias=bias)
    y2 = quant_hip.gemm_fwd(x, t["qweight"], t["qzeros"], t["scales"], None, 128, bias=bias)
    assert torch.equal(y1, y2)
    ref = oracle.matmul_recons(x.cpu().numpy(), layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    ref = ref + bias.float().cpu().numpy()
    err = np.abs(y1.float().cpu().numpy() - ref).max()
    assert err <= 1e-2 * np.abs(ref).max()


@pytest.mark.parametrize("M", [17, 32, 33, 48, 64])
@pytest.mark.parametrize("K,N,gs,act", [(4096, 1024, 128, False), (1408, 256, 128, False), (512, 384, 128, True),
                                        (11008, 256, 128, False)])
def test_gemm_forward_17_to_64_rows(oracle, M, K, N, gs, act):
    """17..64 rows without act-order take the weight-streaming kernel (all row blocks share one pass over the packed
    weights; partial rows of the K splits are added by a second kernel), act-order the tiled kernel; with bias."""
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    layer = oracle.make_layer(K, N, gs, act_order=act, seed=K + N + M)
    t = to_cuda_layer(layer)
    x = oracle.make_activations(M, K, seed=M + 11)
    bias = (np.random.default_rng(M).standard_normal(N) * 0.5).astype(np.float16)
    ref = oracle.matmul_recons(x, layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"]) + bias.astype(np.float32)
    y = quant_hip.gemm_fwd(torch.from_numpy(x).cuda(), t["qweight"], t["qzeros"], t["scales"], t["g_idx"], gs,
                           bias=torch.from_numpy(bias).cuda())
    y2 = quant_hip.gemm_fwd(torch.from_numpy(x).cuda(), t["qweight"], t["qzeros"], t["scales"], t["g_idx"], gs,
                            bias=torch.from_numpy(bias).cuda())
    assert y.shape == (M, N) and torch.equal(y, y2)
    assert np.abs(y.float().cpu().numpy() - ref).max() <= 1e-2 * np.abs(ref).max()


@pytest.mark.parametrize("M", [20, 40, 64])
@pytest.mark.parametrize("K,N", [(4096, 11008), (4096, 16512), (2048, 24704)])
def test_gemm_forward_streaming_kernel_several_strips_per_workgroup(oracle, M, K, N):
    """Wide outputs: a workgroup of the streaming kernel walks over 2 or 3 neighbouring 64-column strips with the
    activations held in registers; 16512 and 24704 columns (258 and 386 strips, 4 and 3 per workgroup) leave the
    last workgroup two strips.  (11008 columns = 172 strips take the whole-reduction kernel: one workgroup per strip.)"""
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    layer = oracle.make_layer(K, N, 128, seed=K + N + M)
    t = to_cuda_layer(layer)
    x = oracle.make_activations(M, K, seed=M + 5)
    ref = oracle.matmul_recons(x, layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    y = quant_hip.gemm_fwd(torch.from_numpy(x).cuda(), t["qweight"], t["qzeros"], t["scales"], None, 128)
    y2 = quant_hip.gemm_fwd(torch.from_numpy(x).cuda(), t["qweight"], t["qzeros"], t["scales"], None, 128)
    assert y.shape == (M, N) and torch.equal(y, y2)
    assert np.abs(y.float().cpu().numpy() - ref).max() <= 1e-2 * np.abs(ref).max()


@pytest.mark.parametrize("M", [65, 96, 100, 128, 129, 192, 200, 256, 300, 512])
@pytest.mark.parametrize("K,N,gs", [(4096, 4096, 128), (1408, 256, 128), (512, 384, 256), (11008, 1024, 128),
                                    (1024, 2048, 1024), (128, 128, 128)])
def test_gemm_forward_65_to_512_rows_whole_reduction_streaming_kernel(oracle, M, K, N, gs):
    """More than 64 rows of an output that one round of workgroups covers: one 64-column strip of 32, 48 or 64 rows per
    workgroup over the whole reduction (11 and 86 chunks of 128: uneven shares of the eight wavefronts; 1 and 4
    chunks: idle wavefronts), activation tiles delivered to LDS by the loads themselves, row blocks cut off by M,
    with bias.  Same dequantized weights as the tiled kernel, which the other shapes of this list still take."""
    import torch
    from alpaca_lora_4bit_amd import _lib, quant_hip
    layer = oracle.make_layer(K, N, gs, seed=K + N + M)
    t = to_cuda_layer(layer)
    x = oracle.make_activations(M, K, seed=M + 13)
    bias = (np.random.default_rng(M).standard_normal(N) * 0.5).astype(np.float16)
    ref = oracle.matmul_recons(x, layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"]) + bias.astype(np.float32)
    y = quant_hip.gemm_fwd(torch.from_numpy(x).cuda(), t["qweight"], t["qzeros"], t["scales"], None, gs,
                           bias=torch.from_numpy(bias).cuda())
    y2 = quant_hip.gemm_fwd(torch.from_numpy(x).cuda(), t["qweight"], t["qzeros"], t["scales"], None, gs,
                            bias=torch.from_numpy(bias).cuda())
    assert y.shape == (M, N) and torch.equal(y, y2)
    assert np.abs(y.float().cpu().numpy() - ref).max() <= 1e-2 * np.abs(ref).max()
    assert np.abs(y.float().cpu().numpy() - ref).max() <= 2e-3 * np.abs(ref).max()
    lib = _lib.lib()
    strips = N // 64
    rb = next((rb for rb in (2, 3, 4) if strips * -(-M // (16 * rb)) <= 256), 0)
    assert bool((lib.q4_gemm_route(1, M, K, N, gs, 0) == 2)) == (rb == 2 or (rb > 2 and K <= 12288))
    assert not (lib.q4_gemm_route(1, M, K, N, gs, 1) == 2) and not (lib.q4_gemm_route(1, 64, K, N, gs, 0) == 2)


@pytest.mark.parametrize("M", [17, 32, 33, 48, 49, 64])
@pytest.mark.parametrize("K,N", [(512, 8192), (1408, 11008), (128, 16384)])
def test_gemm_forward_17_to_64_rows_of_wide_outputs_whole_reduction_streaming_kernel(oracle, M, K, N):
    """17..64 rows of an output with 128..256 strips: one workgroup per strip over the whole reduction (one row block of
    32, 48 or 64 rows), instead of the split reduction with partial rows and a second kernel."""
    import torch
    from alpaca_lora_4bit_amd import _lib, quant_hip
    layer = oracle.make_layer(K, N, 128, seed=K + N + M)
    t = to_cuda_layer(layer)
    x = oracle.make_activations(M, K, seed=M + 19)
    ref = oracle.matmul_recons(x, layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    y = quant_hip.gemm_fwd(torch.from_numpy(x).cuda(), t["qweight"], t["qzeros"], t["scales"], None, 128)
    y2 = quant_hip.gemm_fwd(torch.from_numpy(x).cuda(), t["qweight"], t["qzeros"], t["scales"], None, 128)
    assert y.shape == (M, N) and torch.equal(y, y2)
    assert np.abs(y.float().cpu().numpy() - ref).max() <= 2e-3 * np.abs(ref).max()
    assert _lib.lib().q4_gemm_route(1, M, K, N, 128, 0) == 2


@pytest.mark.parametrize("M", [49, 64, 65, 96, 100, 128, 129, 192, 200, 256, 300, 512])
@pytest.mark.parametrize("K,N,gs", [(4096, 4096, 128), (256, 1408, 128), (384, 512, 128), (1024, 11008, 128),
                                    (2048, 1024, 1024), (128, 128, 128)])
def test_gemm_grad_input_49_to_512_rows_whole_reduction_streaming_kernel(oracle, M, K, N, gs):
    """Grad-input counterpart: one block of 128 outputs of 32 or 48 rows per workgroup over the whole reduction (11 and
    86 chunks of 128 columns: uneven shares of the eight wavefronts; 1 and 4 chunks: idle wavefronts), row blocks cut
    off by M.  Shapes of this list with more row blocks than one round of workgroups holds take the tiled kernel."""
    import torch
    from alpaca_lora_4bit_amd import _lib, quant_hip
    layer = oracle.make_layer(K, N, gs, seed=K + N + M + 1)
    t = to_cuda_layer(layer)
    dy = oracle.make_activations(M, N, seed=M + 17)
    ref = oracle.matmul_recons_t(dy, layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    dx = quant_hip.gemm_bwd_dx(torch.from_numpy(dy).cuda(), t["qweight"], t["qzeros"], t["scales"], None, gs)
    dx2 = quant_hip.gemm_bwd_dx(torch.from_numpy(dy).cuda(), t["qweight"], t["qzeros"], t["scales"], None, gs)
    assert dx.shape == (M, K) and torch.equal(dx, dx2)
    assert np.abs(dx.float().cpu().numpy() - ref).max() <= 1e-2 * np.abs(ref).max()
    assert np.abs(dx.float().cpu().numpy() - ref).max() <= 2e-3 * np.abs(ref).max()
    lib = _lib.lib()
    rb = next((rb for rb in (2, 3) if (K // 128) * -(-M // (16 * rb)) <= 256), 0)
    assert bool((lib.q4_gemm_route(0, M, K, N, gs, 0) == 2)) == (rb != 0 and N <= 2 * K)
    assert not (lib.q4_gemm_route(0, M, K, N, gs, 1) == 2) and not (lib.q4_gemm_route(0, 48, K, N, gs, 0) == 2)


@pytest.mark.parametrize("act", [False, True])
@pytest.mark.parametrize("M,red,nout,tail_cols,tail_splits", [(1024, 1024, 11136, 23, 2), (520, 1024, 11008, 1, 2),
                                                              (1536, 4096, 11008, 1, 8)])
def test_gemm_remainder_tiles_run_as_a_split_second_launch(oracle, M, red, nout, tail_cols, tail_splits, act):
    """More 256-row tiles than CUs with a last round that fills at most half of them: the remainder's column tiles
    go to a second launch with the reduction split; forward (bias + adapter) and backward-dx (adapter) must cover
    every column exactly once."""
    import torch
    from alpaca_lora_4bit_amd import _lib, quant_hip
    r, scaling = 8, 2.0
    for fwd in (True, False):
        K, N = (red, nout) if fwd else (nout, red)
        assert _lib.lib().q4_gemm_workspace_bytes(int(fwd), M, K, N) == tail_splits * M * tail_cols * 128 * 4
        layer = oracle.make_layer(K, N, 128, act_order=act, seed=53)
        t = to_cuda_layer(layer)
        A, B = oracle.make_lora(K, N, r, seed=53)
        A16, B16 = A.astype(np.float16), B.astype(np.float16)
        W = oracle.dequant_v2(layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"]).astype(np.float64)
        x = oracle.make_activations(M, K, seed=43)
        dy = oracle.make_activations(M, N, seed=44)
        if fwd:
            bias = (np.random.default_rng(2).standard_normal(N) * 0.1).astype(np.float16)
            ref = oracle.lora_forward(x, W, A16, B16, scaling, bias=bias)
            xt = _t(x)
            got = quant_hip.gemm_fwd(xt, t["qweight"], t["qzeros"], t["scales"], t["g_idx"], 128, bias=_t(bias),
                                     xa=xt @ _t(A16).t(), lora_bt=_t(B16).t(), lora_scale=scaling)
            plain = quant_hip.gemm_fwd(xt, t["qweight"], t["qzeros"], t["scales"], t["g_idx"], 128)
            ref_plain = x.astype(np.float64) @ W
        else:
            ref, _, _ = oracle.lora_backward(x, dy, W, A16, B16, scaling)
            dyt = _t(dy)
            got = quant_hip.gemm_bwd_dx(dyt, t["qweight"], t["qzeros"], t["scales"], t["g_idx"], 128,
                                        dyb=dyt @ _t(B16), lora_a=_t(A16), lora_scale=scaling)
            plain = quant_hip.gemm_bwd_dx(dyt, t["qweight"], t["qzeros"], t["scales"], t["g_idx"], 128)
            ref_plain = dy.astype(np.float64) @ W.T
        torch.cuda.synchronize()
        for out, want in ((got, ref), (plain, ref_plain)):
            out = out.cpu().numpy()
            assert rel_err(out, want) <= TOL
            edge = (nout // 128 - tail_cols) * 128                  # first column of the second launch
            assert rel_err(out[:, edge - 128:edge + 128], want[:, edge - 128:edge + 128]) <= TOL
            assert rel_err(out[:, -128:], want[:, -128:]) <= TOL


_GRAPH_SCRIPT = r'''
import sys
sys.path.insert(0, sys.argv[1])
import torch
import bench
from alpaca_lora_4bit_amd import quant_hip

gen = torch.Generator(device="cuda").manual_seed(3)
cases = [(300, 1024, 768), (40, 1024, 768), (3072, 512, 3072), (1024, 2048, 1024)]   # split-K, streaming, wide tiles, two-way split
for (M, K, N) in cases:
    lay = bench.make_layer_gpu(K, N, 128, gen, False)
    w = (lay["qweight"], lay["qzeros"], lay["scales"], lay["g_idx"], 128)
    assert quant_hip.scales_fit_fused_dequant(lay["scales"])     # the content check reads back once: before the capture
    x = torch.randn((M, K), device="cuda", generator=gen).half()
    dy = torch.randn((M, N), device="cuda", generator=gen).half()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):         # the first products of this shape are issued under capture
        y = quant_hip.gemm_fwd(x, *w)
        dx = quant_hip.gemm_bwd_dx(dy, *w)
    for rep in range(3):
        x.normal_(generator=gen)
        dy.normal_(generator=gen)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        y_e = quant_hip.gemm_fwd(x, *w)
        dx_e = quant_hip.gemm_bwd_dx(dy, *w)
        torch.cuda.synchronize()
        assert torch.equal(y, y_e) and torch.equal(dx, dx_e), (M, K, N, rep)
        assert float(y.float().abs().max()) > 0 and float(dx.float().abs().max()) > 0
print("graph ok")
'''


def test_products_first_issued_under_graph_capture_replay_like_eager():
    """A fresh process whose very first GEMM launches happen while a HIP graph is being captured (the launchers set a
    kernel attribute on first use; only the per-tensor content check, which reads a value back, ran before): every
    replay, with new inputs and eager work in between, equals the eager call bit for bit."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-c", _GRAPH_SCRIPT, root], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "graph ok" in r.stdout, r.stdout[-2000:] + r.stderr[-4000:]
