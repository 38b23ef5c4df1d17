"""q4_gemv_noalloc_f16 (the entry point for callers that cannot allocate: its split-K accumulators live in a
device array inside the library) against q4_gemv_f16 with a caller workspace, through the C ABI.
Both run the same kernels with a fixed-order integer reduction, so the outputs must be bit-identical; each is also
held to the oracle within 1e-2 * max|ref|."""
import numpy as np
import pytest

from conftest import rel_err, to_cuda_layer

pytestmark = pytest.mark.gpu


def _both(L, t, x, M, K, N, G, use_gidx):
    import torch
    stream = torch.cuda.current_stream().cuda_stream
    gp = t["g_idx"].data_ptr() if use_gidx else None
    nbytes = L.q4_gemv_workspace_bytes(M, K, N)
    ws = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    want = torch.empty((M, N), dtype=torch.float16, device="cuda")
    rc = L.q4_gemv_f16(x.data_ptr(), t["qweight"].data_ptr(), t["qzeros"].data_ptr(), t["scales"].data_ptr(), gp,
                       t["groupsize"], want.data_ptr(), 0, M, K, N, G, ws.data_ptr(), nbytes, stream)
    assert rc == 0
    got = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    rc = L.q4_gemv_noalloc_f16(x.data_ptr(), t["qweight"].data_ptr(), t["qzeros"].data_ptr(), t["scales"].data_ptr(), gp,
                               t["groupsize"], got.data_ptr(), 0, M, K, N, G, stream)
    assert rc == 0
    torch.cuda.synchronize()
    return got.cpu().numpy(), want.cpu().numpy()


def test_noalloc_gemv_matches_workspace_gemv_twice_second_call_smaller(oracle):
    import torch
    from alpaca_lora_4bit_amd import _lib
    L = _lib.lib()
    assert L.q4_gemv_noalloc_max_outputs() == 16 * 32768
    # first a large product (many split-K workgroups per strip), then a smaller one that reuses the front of
    # the same array, then an act-order layer through g_idx
    cases = [(16, 4096, 11008, False, False), (3, 1024, 320, False, False), (1, 11008, 4096, False, False),
             (5, 512, 192, True, True)]
    for M, K, N, act, use_gidx in cases:
        layer = oracle.make_layer(K, N, 128, act_order=act, seed=K + N + M)
        t = to_cuda_layer(layer)
        xh = oracle.make_activations(M, K, seed=M)
        x = torch.from_numpy(xh).cuda()
        got, want = _both(L, t, x, M, K, N, layer["scales"].shape[0], use_gidx)
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), (M, K, N)
        ref = oracle.matmul_recons(xh, layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
        assert rel_err(got, ref) <= 1e-2


def test_noalloc_gemv_repeats_and_accumulates(oracle):
    """Repeated calls on the shared array give the same product every time; accumulate=1 adds to y."""
    import torch
    from alpaca_lora_4bit_amd import _lib
    L = _lib.lib()
    M, K, N = 2, 2048, 256
    layer = oracle.make_layer(K, N, 128, seed=9)
    t = to_cuda_layer(layer)
    xh = oracle.make_activations(M, K, seed=9)
    x = torch.from_numpy(xh).cuda()
    ref = oracle.matmul_recons(xh, layer["qweight"], layer["qzeros"], layer["scales"], layer["g_idx"])
    stream = torch.cuda.current_stream().cuda_stream
    y = torch.full((M, N), 1.5, dtype=torch.float16, device="cuda")
    for rep in range(3):
        y.fill_(1.5)
        rc = L.q4_gemv_noalloc_f16(x.data_ptr(), t["qweight"].data_ptr(), t["qzeros"].data_ptr(), t["scales"].data_ptr(),
                                   None, 128, y.data_ptr(), 1, M, K, N, K // 128, stream)
        assert rc == 0
        torch.cuda.synchronize()
        assert rel_err(y.cpu().numpy(), ref + 1.5) <= 1e-2


def test_noalloc_gemv_rejects_what_does_not_fit():
    import ctypes
    from alpaca_lora_4bit_amd import _lib
    L = _lib.lib()
    fake = ctypes.c_void_p(0x1000)
    # 16 x 32832 accumulators > 524 288: rejected before anything is enqueued (the pointers are never touched)
    assert L.q4_gemv_noalloc_f16(fake, fake, fake, fake, None, 128, fake, 0, 16, 256, 32832, 2, None) == -6
    assert L.q4_gemv_noalloc_f16(fake, fake, fake, fake, None, 128, fake, 0, 17, 256, 128, 2, None) == -2
    assert L.q4_gemv_noalloc_f16(None, fake, fake, fake, None, 128, fake, 0, 1, 256, 128, 2, None) == -1
    assert b"scratch" in L.q4_error_string(-6)


def test_noalloc_gemv_captured_in_a_hip_graph_and_replayed(oracle):
    """What the entry point is for: after one eager call on the device (the address look-up), a call is recorded into
    a HIP graph and replayed several times, with eager work and synchronisations of the program's own in between;
    every replay must give the bits of the eager call."""
    import torch
    from alpaca_lora_4bit_amd import _lib
    L = _lib.lib()
    M, K, N = 4, 4096, 4096
    layer = oracle.make_layer(K, N, 128, seed=21)
    t = to_cuda_layer(layer)
    xs = [torch.from_numpy(oracle.make_activations(M, K, seed=s)).cuda() for s in (1, 2, 3)]
    x = xs[0].clone()
    y = torch.empty((M, N), dtype=torch.float16, device="cuda")

    def call(stream):
        return L.q4_gemv_noalloc_f16(x.data_ptr(), t["qweight"].data_ptr(), t["qzeros"].data_ptr(), t["scales"].data_ptr(),
                                     None, 128, y.data_ptr(), 0, M, K, N, K // 128, stream)

    want = []
    for xi in xs:                                       # eager results (also the first call on the device)
        x.copy_(xi)
        assert call(torch.cuda.current_stream().cuda_stream) == 0
        torch.cuda.synchronize()
        want.append(y.clone())
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        assert call(torch.cuda.current_stream().cuda_stream) == 0
    for rep in range(6):
        xi = xs[rep % 3]
        x.copy_(xi)
        y.fill_(float("nan"))
        (xi.float() @ xi.float().t()).sum().item()      # eager work and a host read between two replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want[rep % 3]), rep
