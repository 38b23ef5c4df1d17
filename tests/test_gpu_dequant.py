"""HIP dense dequant vs the CPU oracle: BIT-EXACT (integer compare of the fp16 patterns)."""
import numpy as np
import pytest

from conftest import to_cuda_layer

pytestmark = pytest.mark.gpu


def _run(layer, use_gidx=True):
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    t = to_cuda_layer(layer)
    W = quant_hip.dequant(t["qweight"], t["qzeros"], t["scales"], t["g_idx"] if use_gidx else None, t["groupsize"])
    torch.cuda.synchronize()
    return W.cpu().numpy()


@pytest.mark.parametrize("K,N,gs,act", [
    (256, 128, 128, False), (256, 128, 128, True), (64, 64, 32, False), (512, 192, 64, True),
    (4096, 4096, 128, False),          # benchmark config 0
    (4096, 11008, 128, False),         # config 1 gate/up
    (11008, 4096, 128, False),         # config 1 down
    (5120, 13824, 128, True),          # config 3 act-order
    (1024, 256, 1024, False),          # one group (groupsize = -1 case)
])
def test_dequant_bit_exact(oracle, K, N, gs, act):
    layer = oracle.make_layer(K, N, gs, act_order=act, seed=K + N)
    ref = oracle.dequant_v2(layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    got = _run(layer)
    assert np.array_equal(got.view(np.uint16), ref.view(np.uint16))
    if not act:
        got2 = _run(layer, use_gidx=False)      # g_idx == NULL path of the C ABI
        assert np.array_equal(got2.view(np.uint16), ref.view(np.uint16))


@pytest.mark.parametrize("case", ["seq", "actorder"])
def test_hip_paths_match_committed_golden_fixture(case):
    """Dequant bit-exact, GEMV / GEMM forward / GEMM backward within 1e-2 of the exact-rational
    expectations in tests/golden/q4_golden.npz (made without any code from oracle/)."""
    import os
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    from conftest import rel_err
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "q4_golden.npz"))
    t = {k: torch.from_numpy(gold[f"{case}_{k}"]).cuda() for k in ("qweight", "qzeros", "scales", "g_idx", "x", "dy")}
    W = quant_hip.dequant(t["qweight"], t["qzeros"], t["scales"], t["g_idx"], 128)
    assert np.array_equal(W.cpu().numpy().view(np.uint16), gold[f"{case}_W_bits"])
    y = quant_hip.gemv(t["x"], t["qweight"], t["qzeros"], t["scales"], t["g_idx"], 128)
    assert rel_err(y.cpu().numpy(), gold[f"{case}_y"]) <= 1e-2
    y2 = quant_hip.gemm_fwd(t["x"], t["qweight"], t["qzeros"], t["scales"], t["g_idx"], 128)
    assert rel_err(y2.cpu().numpy(), gold[f"{case}_y"]) <= 1e-2
    dx = quant_hip.gemm_bwd_dx(t["dy"], t["qweight"], t["qzeros"], t["scales"], t["g_idx"], 128)
    assert rel_err(dx.cpu().numpy(), gold[f"{case}_dx"]) <= 1e-2


def test_dequant_exhaustive_scalar_table(oracle):
    """Every finite fp16 scale x 16 codes x 16 zero codes (16.25 M cases) through the HIP kernel."""
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    finite = bits[np.isfinite(bits.view(np.float16))]
    n_s = finite.size                                   # 63488
    N = ((n_s + 63) // 64) * 64
    scales_row = np.zeros(N, dtype=np.uint16)
    scales_row[:n_s] = finite
    G = 16                                              # group g has zero code g in every column
    K = 16 * 32                                         # 32 rows per group; code of row k is k % 16
    scales = np.tile(scales_row.view(np.float16), (G, 1))
    zcodes = np.repeat(np.arange(G, dtype=np.uint8)[:, None], N, axis=1)
    codes = np.repeat((np.arange(K) % 16).astype(np.uint8)[:, None], N, axis=1)
    g_idx = (np.arange(K) // 32).astype(np.int32)
    qweight, qzeros = oracle.pack_qweight(codes), oracle.pack_qzeros(zcodes)
    with np.errstate(all="ignore"):
        ref = oracle.dequant_v2(qweight, qzeros, scales, g_idx)
    W = quant_hip.dequant(torch.from_numpy(qweight).cuda(), torch.from_numpy(qzeros).cuda(),
                          torch.from_numpy(scales).cuda(), torch.from_numpy(g_idx).cuda(), 32)
    got = W.cpu().numpy()
    same = (got.view(np.uint16) == ref.view(np.uint16)) | (np.isnan(got) & np.isnan(ref))
    assert same[:, :n_s].all(), f"{(~same[:, :n_s]).sum()} mismatches"


def test_dequant_distinguishes_rounding_orders(oracle):
    """The single-rounding form (q-(z+1))*s differs from the reference's three roundings in a
    large fraction of elements; the kernel must match the latter, not the former."""
    layer = oracle.make_layer(512, 256, 128, seed=5)
    three = oracle.dequant_v2(layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    one = oracle.dequant_v2_single_rounding(layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    assert (three.view(np.uint16) != one.view(np.uint16)).mean() > 0.2
    got = _run(layer)
    assert np.array_equal(got.view(np.uint16), three.view(np.uint16))


def test_quant_cuda_compatible_recons(oracle):
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    layer = oracle.make_layer(256, 128, 128, act_order=True, seed=9)
    t = to_cuda_layer(layer)
    res = torch.zeros((256, 128), dtype=torch.float16, device="cuda")
    assert quant_hip.vecquant4recons_v2(t["qweight"], res, t["scales"], t["qzeros"], t["g_idx"]) is None
    ref = oracle.dequant_v2(layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    assert np.array_equal(res.cpu().numpy().view(np.uint16), ref.view(np.uint16))


def test_dequant_rejects_bad_arguments(oracle):
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    layer = oracle.make_layer(256, 128, 128, seed=1)
    t = to_cuda_layer(layer)
    with pytest.raises(ValueError):
        quant_hip.dequant(t["qweight"], t["qzeros"], t["scales"].float(), t["g_idx"], 128)
    with pytest.raises(ValueError):
        quant_hip.dequant(t["qweight"], t["qzeros"][:, :8].contiguous(), t["scales"], t["g_idx"], 128)
    bad = t["g_idx"].clone()
    bad[3] = 99
    with pytest.raises(ValueError):
        quant_hip.dequant(t["qweight"], t["qzeros"], t["scales"], bad, 128)


# --------------------------------------------------------------------------- float flavour (fp32 scales, fp32 W)
def test_dequant_f32_matches_committed_golden_fixture():
    """Bit-exact with tests/golden/q4_golden_f32.npz (exact rational arithmetic, made without oracle/): the table of
    every (q, z) for 228 scale patterns through the kernel, and an act-order layer."""
    import os
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    from test_oracle import _scalar_layer_f32, _scalar_table_of
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "q4_golden_f32.npz"))
    qw, qz, scales, g_idx, n = _scalar_layer_f32()
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    for gi in (dev(g_idx), None):                                # gathered and sequential group lookup
        W = quant_hip.dequant_f32(dev(qw), dev(qz), dev(scales), gi, 32)
        got = _scalar_table_of(W.cpu().numpy().view(np.uint32), n)
        exp = gold["scalar_fused"]
        assert ((got == exp) | (((got | exp) & 0x7FFFFFFF) == 0)).all()
    W = quant_hip.dequant_f32(dev(gold["layer_qweight"]), dev(gold["layer_qzeros"]), dev(gold["layer_scales"]),
                              dev(gold["layer_g_idx"]), 32)
    assert np.array_equal(W.cpu().numpy().view(np.uint32), gold["layer_W_bits"])


@pytest.mark.parametrize("K,N,gs,act", [(256, 128, 128, True), (4096, 4096, 128, False), (5120, 13824, 128, True),
                                        (11008, 4096, 128, False)])
def test_dequant_f32_bit_exact_with_oracle_and_through_the_quant_cuda_name(oracle, K, N, gs, act):
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    layer = oracle.make_layer(K, N, gs, act_order=act, seed=K + N + 1)
    rng = np.random.default_rng(K)
    scales = (layer["scales"].astype(np.float32) * rng.uniform(0.9, 1.1, size=layer["scales"].shape)).astype(np.float32)
    ref = oracle.dequant_v2_f32(layer["qweight"], layer["qzeros"], scales, layer["g_idx"])
    t = to_cuda_layer(layer)
    res = torch.zeros((K, N), dtype=torch.float32, device="cuda")
    assert quant_hip.vecquant4recons_v2(t["qweight"], res, torch.from_numpy(scales).cuda(), t["qzeros"], t["g_idx"]) is None
    assert np.array_equal(res.cpu().numpy().view(np.uint32), ref.view(np.uint32))
    with pytest.raises(ValueError):                              # the reference reads `res` as the scales' type
        quant_hip.vecquant4recons_v2(t["qweight"], res.half(), torch.from_numpy(scales).cuda(), t["qzeros"], t["g_idx"])
    # fp32 copies of fp16 scales still give the fp16 kernel's values when `res` is fp16-typed storage of the module path
    W16 = quant_hip.dequant(t["qweight"], t["qzeros"], t["scales"], t["g_idx"], gs)
    W32 = quant_hip.dequant_f32(t["qweight"], t["qzeros"], t["scales"].float(), t["g_idx"], gs)
    assert (W32 - W16.float()).abs().max().item() <= 2.0 ** -9 * W16.abs().max().item()     # fp16 roundings only
