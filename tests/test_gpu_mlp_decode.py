"""Fused MLP decode step (q4_mlp_decode_f16: gate|up -> silu * up -> down in one launch) vs the CPU oracle and vs
the three separate products.  Tolerance for y: max|y - ref| <= 1e-2 * max|ref| against the float64 result computed
from the oracle's dequantized weights with the intermediate rounded to fp16 where the unfused modules round it."""
import ctypes

import numpy as np
import pytest

from conftest import rel_err, to_cuda_layer

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _layers(oracle, H, I, gs, seed):
    gate = oracle.make_layer(H, I, gs, seed=seed)
    up = oracle.make_layer(H, I, gs, seed=seed + 1)
    down = oracle.make_layer(I, H, gs, seed=seed + 2)
    return gate, up, down


def _dense(oracle, layer):
    return oracle.dequant_v2(layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"]).astype(np.float64)


def _reference(oracle, x, gate, up, down):
    """float64 products; fp16 roundings of gate, up, silu(gate) and the product, as the modules apply them."""
    g = (x.astype(np.float64) @ _dense(oracle, gate)).astype(np.float16)
    u = (x.astype(np.float64) @ _dense(oracle, up)).astype(np.float16)
    g32 = g.astype(np.float32)
    h = (g32 / (1.0 + np.exp(-g32))).astype(np.float16)
    inter = (h.astype(np.float32) * u.astype(np.float32)).astype(np.float16)
    return g, u, inter, inter.astype(np.float64) @ _dense(oracle, down)


def _tuple(t):
    return (t["qweight"], t["qzeros"], t["scales"])


@pytest.mark.parametrize("H,I,gs", [(4096, 11008, 128), (256, 384, 128), (128, 128, 128), (512, 1408, 128),
                                    (1024, 2816, 256), (2048, 1024, 1024)])
@pytest.mark.parametrize("M", [1, 3, 4, 16])
def test_mlp_decode_matches_oracle_and_separate_products(oracle, H, I, gs, M):
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    gate, up, down = _layers(oracle, H, I, gs, seed=H + I + M)
    tg, tu, td = (to_cuda_layer(l) for l in (gate, up, down))
    x = oracle.make_activations(M, H, seed=M + 5)
    xt = torch.from_numpy(x).cuda()
    g_ref, u_ref, inter_ref, y_ref = _reference(oracle, x, gate, up, down)

    y, g, u = quant_hip.mlp_decode(xt, _tuple(tg), _tuple(tu), _tuple(td), gs, intermediates=True)
    assert y.shape == (M, H) and g.shape == (M, I) and u.shape == (M, I)
    assert rel_err(g.cpu().numpy(), g_ref.astype(np.float64)) <= 2e-3
    assert rel_err(u.cpu().numpy(), u_ref.astype(np.float64)) <= 2e-3
    assert rel_err(y.cpu().numpy(), y_ref) <= TOL, rel_err(y.cpu().numpy(), y_ref)
    assert rel_err(y.cpu().numpy(), y_ref) <= 3e-3

    # the two projections are the GEMV's values (the same bits when K is long enough for the same eight-wavefront
    # split, one fp16 rounding apart otherwise); the output agrees with the unfused chain
    g2 = quant_hip.gemv(xt, tg["qweight"], tg["qzeros"], tg["scales"], None, gs)
    u2 = quant_hip.gemv(xt, tu["qweight"], tu["qzeros"], tu["scales"], None, gs)
    if H >= 1024:
        assert torch.equal(g, g2) and torch.equal(u, u2)
    assert rel_err(g.cpu().numpy(), g2.float().cpu().numpy().astype(np.float64)) <= 1e-3
    assert rel_err(u.cpu().numpy(), u2.float().cpu().numpy().astype(np.float64)) <= 1e-3
    y2 = quant_hip.gemv(torch.nn.functional.silu(g2) * u2, td["qweight"], td["qzeros"], td["scales"], None, gs)
    assert rel_err(y.cpu().numpy(), y2.float().cpu().numpy().astype(np.float64)) <= 3e-3

    # every launch advances the ticket; results do not depend on it, with or without the intermediates
    for _ in range(4):
        assert torch.equal(y, quant_hip.mlp_decode(xt, _tuple(tg), _tuple(tu), _tuple(td), gs))
    assert not quant_hip.mlp_decode_gave_up()
    assert quant_hip.workspaces_are_zero()


def test_mlp_decode_many_launches_back_to_back_and_changing_inputs(oracle):
    """300 launches on one workspace without a synchronisation in between, inputs alternating between two tensors:
    a consumer never picks up a word of an earlier launch (the tag in the hand-over words) and the accumulators end
    at zero every time."""
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    H, I, gs = 1024, 2816, 128
    gate, up, down = _layers(oracle, H, I, gs, seed=77)
    tg, tu, td = (to_cuda_layer(l) for l in (gate, up, down))
    xs = [torch.from_numpy(oracle.make_activations(2, H, seed=s)).cuda() for s in (1, 2)]
    want = [quant_hip.mlp_decode(x, _tuple(tg), _tuple(tu), _tuple(td), gs).clone() for x in xs]
    for x, w in zip(xs, want):
        ref = _reference(oracle, x.cpu().numpy(), gate, up, down)[3]
        assert rel_err(w.cpu().numpy(), ref) <= 3e-3
    outs = [quant_hip.mlp_decode(xs[i & 1], _tuple(tg), _tuple(tu), _tuple(td), gs) for i in range(300)]
    torch.cuda.synchronize()
    for i, o in enumerate(outs):
        assert torch.equal(o, want[i & 1]), i
    assert not quant_hip.mlp_decode_gave_up()


def test_mlp_decode_through_the_c_abi_and_in_a_hip_graph(oracle):
    """Direct call of q4_mlp_decode_f16 with a caller-owned zeroed workspace; the same call captured in a HIP graph and
    replayed (the ticket lives in device memory, so replays of identical launch arguments still get fresh tags)."""
    import torch
    from alpaca_lora_4bit_amd import _lib, quant_hip
    H, I, gs, M = 512, 1408, 128, 4
    gate, up, down = _layers(oracle, H, I, gs, seed=5)
    tg, tu, td = (to_cuda_layer(l) for l in (gate, up, down))
    x = torch.from_numpy(oracle.make_activations(M, H, seed=9)).cuda()
    want = quant_hip.mlp_decode(x, _tuple(tg), _tuple(tu), _tuple(td), gs)
    L = _lib.lib()
    need = L.q4_mlp_decode_workspace_bytes(M, H, I)
    assert need >= 8 * M * (2 * I + H) + 8 * M * I
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    y = torch.empty(M, H, dtype=torch.float16, device="cuda")
    desc = [_lib.Layer(t["qweight"].data_ptr(), t["qzeros"].data_ptr(), t["scales"].data_ptr()) for t in (tg, tu, td)]

    def call(stream):
        return L.q4_mlp_decode_f16(x.data_ptr(), ctypes.byref(desc[0]), ctypes.byref(desc[1]), ctypes.byref(desc[2]), gs,
                                   None, None, y.data_ptr(), M, H, I, ws.data_ptr(), need, stream)

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        assert call(side.cuda_stream) == 0
        side.synchronize()
        assert torch.equal(y, want)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            assert call(torch.cuda.current_stream().cuda_stream) == 0
            assert call(torch.cuda.current_stream().cuda_stream) == 0
    for _ in range(5):
        y.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want)
    off = L.q4_mlp_decode_status_offset(M, H, I)
    assert int(ws[off:off + 4].view(torch.int32).item()) == 0
    # argument validation
    assert L.q4_mlp_decode_f16(x.data_ptr(), ctypes.byref(desc[0]), ctypes.byref(desc[1]), ctypes.byref(desc[2]), gs,
                               None, None, y.data_ptr(), M, H, I, ws.data_ptr(), need - 1, None) == -3
    assert L.q4_mlp_decode_f16(x.data_ptr(), ctypes.byref(desc[0]), ctypes.byref(desc[1]), ctypes.byref(desc[2]), 64,
                               None, None, y.data_ptr(), M, H, I, ws.data_ptr(), need, None) == -2
    assert L.q4_mlp_decode_f16(None, ctypes.byref(desc[0]), ctypes.byref(desc[1]), ctypes.byref(desc[2]), gs,
                               None, None, y.data_ptr(), M, H, I, ws.data_ptr(), need, None) == -1
