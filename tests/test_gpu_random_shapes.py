"""Seeded sweep over random shapes: every matmul entry (GEMV, streaming and tiled forward, grad-input) against
torch.matmul on the library's own bit-exact dense W.  Complements the fixed-shape oracle tests: it is there to catch
indexing mistakes at odd combinations of rows, reduction length, column count, group size and act-order."""
import random

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

ROWS = [1, 2, 3, 4, 5, 7, 8, 15, 16, 17, 20, 31, 32, 33, 40, 47, 48, 49, 63, 64, 65, 100, 128, 129, 200, 255, 256, 257,
        300, 511, 513, 777]


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_random_shapes_against_dense_matmul(seed, oracle):
    from alpaca_lora_4bit_amd import quant_hip
    rnd = random.Random(seed)
    g = torch.Generator().manual_seed(100 + seed)
    for case in range(20):
        K = 128 * rnd.choice([1, 2, 3, 4, 5, 8, 11, 16, 32, 43])
        N = 128 * rnd.choice([1, 2, 3, 4, 5, 8, 9, 32, 33])
        gs = rnd.choice([v for v in (32, 64, 128, 256, 512, K) if K % v == 0])
        act = rnd.random() < 0.25
        M = rnd.choice(ROWS)
        G = K // gs
        qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 8, N), dtype=torch.int32, generator=g).cuda()
        qz = torch.randint(-2 ** 31, 2 ** 31 - 1, (G, N // 8), dtype=torch.int32, generator=g).cuda()
        sc = (torch.rand(G, N, generator=g) * 0.015 + 0.005).half().cuda()
        if act:
            perm = torch.randperm(K, generator=g)
            gi = torch.empty(K, dtype=torch.int32)
            gi[perm] = (torch.arange(K) // gs).int()
            gi = gi.cuda()
        else:
            gi = (torch.arange(K) // gs).int().cuda()
        x = torch.randn(M, K, generator=g).half().cuda()
        dy = torch.randn(M, N, generator=g).half().cuda()
        bias = torch.randn(N, generator=g).half().cuda() if rnd.random() < 0.5 else None
        tag = f"seed {seed} case {case}: M={M} K={K} N={N} gs={gs} act={act} bias={bias is not None}"
        W = quant_hip.dequant(qw, qz, sc, gi, gs).float()
        gidx = gi if (act or gs % 64) else None          # the tiled kernels take sequential groups of 64+ rows
        got = {"fwd": (quant_hip.gemm_fwd(x, qw, qz, sc, gidx, gs, bias=bias),
                       x.float() @ W + (bias.float() if bias is not None else 0)),
               "bwd": (quant_hip.gemm_bwd_dx(dy, qw, qz, sc, gidx, gs), dy.float() @ W.t())}
        if M <= 16:
            got["gemv"] = (quant_hip.gemv(x, qw, qz, sc, gi if act else None, gs), x.float() @ W)
        for name, (y, ref) in got.items():
            assert y.shape == ref.shape, (tag, name)
            err = float((y.float() - ref).abs().max() / ref.abs().max())
            assert err <= 3e-3, (tag, name, err)
        # two rows of every case against the CPU oracle itself (its own unpacking and dense W, float64)
        rows = sorted({0, M - 1})
        lay = (qw.cpu().numpy(), qz.cpu().numpy(), sc.cpu().numpy(), gi.cpu().numpy())
        oy = oracle.matmul_recons(x.cpu().numpy()[rows], *lay) + (bias.float().cpu().numpy() if bias is not None else 0)
        odx = oracle.matmul_recons_t(dy.cpu().numpy()[rows], *lay)
        for name, y, ref in (("fwd", got["fwd"][0], oy), ("bwd", got["bwd"][0], odx)):
            err = float(np.abs(y.float().cpu().numpy()[rows] - ref).max() / np.abs(ref).max())
            assert err <= 3e-3, (tag, name, "oracle", err)


@pytest.mark.parametrize("K,gs", [(1408, 256), (1408, 512), (11008, 1024), (640, 512)])
def test_last_group_partial(K, gs):
    """K not a multiple of the group size: ceil(K / gs) groups, the last one partial.  Every row count takes the
    same layer through another kernel (GEMV up to 16 rows, the streaming kernel up to 64, tiles above), and all of
    them must agree with the dense product."""
    from alpaca_lora_4bit_amd import quant_hip
    g = torch.Generator().manual_seed(K + gs)
    N = 384
    G = -(-K // gs)
    qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 8, N), dtype=torch.int32, generator=g).cuda()
    qz = torch.randint(-2 ** 31, 2 ** 31 - 1, (G, N // 8), dtype=torch.int32, generator=g).cuda()
    sc = (torch.rand(G, N, generator=g) * 0.015 + 0.005).half().cuda()
    gi = (torch.arange(K) // gs).int().cuda()
    W = quant_hip.dequant(qw, qz, sc, gi, gs).float()
    # the rows of the partial group carry weight: a kernel that drops them is far off
    assert float(W[(K // gs) * gs:].abs().max()) > 0
    for M in (1, 16, 17, 33, 64, 65, 130):
        x = torch.randn(M, K, generator=g).half().cuda()
        dy = torch.randn(M, N, generator=g).half().cuda()
        ref = x.float() @ W
        outs = {"fwd": quant_hip.gemm_fwd(x, qw, qz, sc, None, gs), "fwd_gidx": quant_hip.gemm_fwd(x, qw, qz, sc, gi, gs)}
        if M <= 16:
            outs["gemv"] = quant_hip.gemv(x, qw, qz, sc, None, gs)
        for name, y in outs.items():
            err = float((y.float() - ref).abs().max() / ref.abs().max())
            assert err <= 3e-3, (K, gs, M, name, err)
        dx = quant_hip.gemm_bwd_dx(dy, qw, qz, sc, None, gs)
        refx = dy.float() @ W.t()
        assert float((dx.float() - refx).abs().max() / refx.abs().max()) <= 3e-3, (K, gs, M, "bwd")
