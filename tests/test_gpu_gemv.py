"""HIP GEMV (M <= 16) vs the CPU oracle.  Tolerance: max|y - ref| <= 1e-2 * max|ref| against
the fp32-accumulated reference result."""
import numpy as np
import pytest

from conftest import rel_err, to_cuda_layer

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _gemv(layer, x, use_gidx=True):
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    t = to_cuda_layer(layer)
    y = quant_hip.gemv(torch.from_numpy(x).cuda(), t["qweight"], t["qzeros"], t["scales"],
                       t["g_idx"] if use_gidx else None, t["groupsize"])
    torch.cuda.synchronize()
    return y.cpu().numpy()


@pytest.mark.parametrize("K,N,gs", [(4096, 4096, 128), (4096, 11008, 128), (11008, 4096, 128),
                                    (256, 128, 128), (64, 64, 32), (1024, 320, 64), (2048, 192, 2048)])
@pytest.mark.parametrize("M", [1, 4, 16])
def test_gemv_sequential_groups(oracle, K, N, gs, M):
    layer = oracle.make_layer(K, N, gs, seed=K * 7 + N)
    x = oracle.make_activations(M, K, seed=M)
    ref = oracle.matmul_recons(x, layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    for use_gidx in (True, False):
        got = _gemv(layer, x, use_gidx)
        assert got.shape == (M, N)
        assert rel_err(got, ref) <= TOL, (use_gidx, rel_err(got, ref))
    # typical error is far below the tolerance: fp32 accumulation, fp16 output rounding only
    assert rel_err(got, ref) <= 2e-3


@pytest.mark.parametrize("K,N,M", [(5120, 13824, 1), (5120, 13824, 16), (256, 128, 3), (512, 192, 7)])
def test_gemv_act_order(oracle, K, N, M):
    layer = oracle.make_layer(K, N, 128, act_order=True, seed=K + 3 * N)
    x = oracle.make_activations(M, K, seed=M + 11)
    ref = oracle.matmul_recons(x, layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    got = _gemv(layer, x)
    assert rel_err(got, ref) <= TOL
    ref32 = oracle.gemv_v2_fp32(x, layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    assert rel_err(got, ref32) <= TOL


def test_gemv_repeatable_and_workspace_left_clean(oracle):
    """The split-K reduction adds partials in a fixed order: repeated calls are bit-identical,
    and the counters in the workspace are back to zero after every call."""
    layer = oracle.make_layer(4096, 4096, 128, seed=2)
    x = oracle.make_activations(4, 4096, seed=2)
    a = _gemv(layer, x)
    for _ in range(5):
        assert np.array_equal(a.view(np.uint16), _gemv(layer, x).view(np.uint16))
    from alpaca_lora_4bit_amd import quant_hip
    assert quant_hip.workspaces_are_zero()


def test_gemv_linearity_full_size(oracle):
    """Size-independent property at a full benchmark shape: (a*x1 + x2) @ W == a*(x1 @ W) + x2 @ W."""
    layer = oracle.make_layer(4096, 11008, 128, seed=4)
    x1 = oracle.make_activations(1, 4096, seed=21)
    x2 = oracle.make_activations(1, 4096, seed=22)
    xs = (2.0 * x1.astype(np.float32) + x2.astype(np.float32)).astype(np.float16)
    y1, y2, ys = _gemv(layer, x1), _gemv(layer, x2), _gemv(layer, xs)
    lin = 2.0 * y1.astype(np.float32) + y2.astype(np.float32)
    assert rel_err(ys, lin) <= 5e-3


def test_quant_cuda_compatible_matmuls(oracle):
    """vecquant4matmul / _faster / _old_faster: accumulate into a pre-zeroed `mul` in its dtype."""
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    layer = oracle.make_layer(512, 256, 128, seed=8)
    t = to_cuda_layer(layer)
    x = oracle.make_activations(2, 512, seed=8)
    ref = oracle.matmul_recons(x, layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    xt = torch.from_numpy(x).cuda()
    y32 = torch.zeros((2, 256), dtype=torch.float32, device="cuda")
    quant_hip.vecquant4matmul(xt.float(), t["qweight"], y32, t["scales"].float(), t["qzeros"], t["g_idx"])
    assert rel_err(y32.cpu().numpy(), ref) <= TOL
    y32.zero_()
    quant_hip.vecquant4matmul_old_faster(xt, t["qweight"], y32, t["scales"].float(), t["qzeros"], 128, 256)
    assert rel_err(y32.cpu().numpy(), ref) <= TOL
    y16 = torch.zeros((2, 256), dtype=torch.float16, device="cuda")
    quant_hip.vecquant4matmul_faster(xt, t["qweight"], y16, t["scales"], t["qzeros"], t["g_idx"], 256)
    assert rel_err(y16.cpu().numpy(), ref) <= TOL
    quant_hip.vecquant4matmul_faster(xt, t["qweight"], y16, t["scales"], t["qzeros"], t["g_idx"], 256)
    assert rel_err(y16.cpu().numpy(), 2 * ref) <= TOL      # second call accumulated


def test_gemv_accumulate_flag(oracle):
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    layer = oracle.make_layer(4096, 256, 128, seed=3)
    t = to_cuda_layer(layer)
    x = oracle.make_activations(3, 4096, seed=3)
    ref = oracle.matmul_recons(x, layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    base = torch.full((3, 256), 1.5, dtype=torch.float16, device="cuda")
    quant_hip.gemv(torch.from_numpy(x).cuda(), t["qweight"], t["qzeros"], t["scales"], None, 128, out=base,
                   accumulate=True)
    assert rel_err(base.cpu().numpy(), ref + 1.5) <= TOL


def test_two_streams_and_two_threads_use_separate_workspaces(oracle):
    """The split-K accumulators (GEMV) and partial-sum scratch (GEMM) are cached per stream: products launched
    concurrently on two streams, from two Python threads, give the bits of the same products run one by one."""
    import threading
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    layers = [to_cuda_layer(oracle.make_layer(4096, 2048, 128, seed=50 + i)) for i in range(2)]
    xs = [torch.from_numpy(oracle.make_activations(m, 4096, seed=60 + i)).cuda() for i, m in enumerate((1, 16))]
    xg = [torch.from_numpy(oracle.make_activations(40, 4096, seed=70 + i)).cuda() for i in range(2)]
    want = [quant_hip.gemv(x, t["qweight"], t["qzeros"], t["scales"], None, 128) for x, t in zip(xs, layers)]
    want_g = [quant_hip.gemm_fwd(x, t["qweight"], t["qzeros"], t["scales"], None, 128) for x, t in zip(xg, layers)]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    got = [[None] * 30, [None] * 30]
    got_g = [[None] * 30, [None] * 30]

    def work(i):
        with torch.cuda.stream(streams[i]):
            for r in range(30):
                got[i][r] = quant_hip.gemv(xs[i], layers[i]["qweight"], layers[i]["qzeros"], layers[i]["scales"], None, 128)
                got_g[i][r] = quant_hip.gemm_fwd(xg[i], layers[i]["qweight"], layers[i]["qzeros"], layers[i]["scales"],
                                                 None, 128)
    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    torch.cuda.synchronize()
    for i in range(2):
        assert all(torch.equal(y, want[i]) for y in got[i])
        assert all(torch.equal(y, want_g[i]) for y in got_g[i])


@pytest.mark.parametrize("M", [1, 3, 16])
@pytest.mark.parametrize("K,Ns,gs", [(4096, (11008, 11008), 128), (4096, (4096, 1024, 1024), 128), (512, (64, 192, 128, 320), 64),
                                     (11008, (4096,), 128), (256, (128, 64), 32)])
def test_gemv_grouped_matches_single_launches_and_oracle(oracle, K, Ns, gs, M):
    """q4_gemv_grouped_f16: several layers in one launch, each read from its own tensors.  Same kernels and the same
    fixed-order integer reduction as q4_gemv_f16, so each output is bit-identical to the single-layer launch;
    both are held to the oracle."""
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    layers = [oracle.make_layer(K, N, gs, seed=K + 5 * N + i) for i, N in enumerate(Ns)]
    ts = [to_cuda_layer(l) for l in layers]
    xh = oracle.make_activations(M, K, seed=M + 3)
    x = torch.from_numpy(xh).cuda()
    outs = quant_hip.gemv_grouped(x, [(t["qweight"], t["qzeros"], t["scales"]) for t in ts], gs)
    torch.cuda.synchronize()
    assert len(outs) == len(Ns)
    for lay, t, y in zip(layers, ts, outs):
        single = quant_hip.gemv(x, t["qweight"], t["qzeros"], t["scales"], None, gs)
        assert torch.equal(y, single)
        ref = oracle.matmul_recons(xh, lay["qweight"], lay["qzeros"], lay["scales"], lay["g_idx"])
        assert rel_err(y.cpu().numpy(), ref) <= TOL
    # one activation tensor per layer, g_idx given (sequential), accumulate into existing outputs
    xs = [torch.from_numpy(oracle.make_activations(M, K, seed=40 + i)).cuda() for i in range(len(Ns))]
    base = [torch.full((M, N), 0.5, dtype=torch.float16, device="cuda") for N in Ns]
    quant_hip.gemv_grouped(xs, [(t["qweight"], t["qzeros"], t["scales"], t["g_idx"]) for t in ts], gs, outs=base,
                           accumulate=True)
    for lay, xi, y in zip(layers, xs, base):
        ref = oracle.matmul_recons(xi.cpu().numpy(), lay["qweight"], lay["qzeros"], lay["scales"], lay["g_idx"]) + 0.5
        assert rel_err(y.cpu().numpy(), ref) <= TOL
    assert quant_hip.workspaces_are_zero()                    # accumulators left zeroed


def test_gemv_grouped_rejects_act_order_and_mismatched_layers(oracle):
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    a = to_cuda_layer(oracle.make_layer(256, 128, 128, act_order=True, seed=1))
    b = to_cuda_layer(oracle.make_layer(512, 128, 128, seed=2))
    c = to_cuda_layer(oracle.make_layer(256, 128, 128, seed=3))
    x = torch.zeros((1, 256), dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError):
        quant_hip.gemv_grouped(x, [(a["qweight"], a["qzeros"], a["scales"], a["g_idx"])], 128)
    with pytest.raises(ValueError):
        quant_hip.gemv_grouped(x, [(c["qweight"], c["qzeros"], c["scales"]), (b["qweight"], b["qzeros"], b["scales"])], 128)
    with pytest.raises(ValueError):
        quant_hip.gemv_grouped(x, [(c["qweight"], c["qzeros"], c["scales"])] * 5, 128)
