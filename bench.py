#!/usr/bin/env python3
"""Benchmark of the 4-bit GPTQ dequant-matmul path on one MI355X.

Headline workload (configs[1] of the benchmark definition): LLaMA-7B MLP decode GEMVs at M=1 -- gate and up
4096->11008, down 11008->4096, groupsize 128, no act-order.  One STEP = one token through the
MLP GEMVs of all 32 decoder layers (64 launches: gate|up as one grouped launch + down, over 2.25 GB of DISTINCT packed weights, so
nothing is served from the 256 MB Infinity Cache, exactly as in a real decode).  The step is
captured once in a HIP graph and replayed; inputs and weights are resident in HBM.

Prints ONE JSON line.  `value` = algorithmic bytes of a step / wall time per step (GB/s).
`roofline` is for the dominant kernel (the GEMV): algorithmic bytes of one launch / average
launch duration measured with events on the launch stream.  `cpu_baseline` times the torch-CPU
restatement of the reference's recons+matmul algorithm on a bounded sample.
Secondary figures (M=4/16, config 0, the config-2 LoRA fwd+bwd step, config 3) go under "extra".
"""
import argparse
import contextlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, GB/s
MFMA_FP16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 MFMA
# HBM bytes per launch of the headline kernel (the grouped gate|up GEMV), measured in two rocprofv3 --pmc runs
# (FETCH_SIZE, WRITE_SIZE), each scaled by what the same counter reads for a 256 MiB copy (--calibrate-copy):
# 2 x 23 470.3 KiB read + 903.0 KiB written.  Not re-measured by a bench run: the file named below holds the commands.
GEMV_TRAFFIC_BYTES = 48991000
GEMV_TRAFFIC_SOURCE = "profiles/gemv_mlp_decode_M1_gate_up_grouped_and_down.md"


def gemv_bytes(M, K, N, G, act_order=False):
    """Algorithmic bytes of one GEMV launch: packed weights + zeros + scales (+ g_idx) + x + y."""
    return K * N // 2 + G * N // 2 + 2 * G * N + (4 * K if act_order else 0) + 2 * M * K + 2 * M * N


def make_layer_gpu(K, N, gs, gen, act_order=False):
    import torch
    G = (K + gs - 1) // gs
    dev = "cuda"
    lay = dict(
        qweight=torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 8, N), dtype=torch.int32, device=dev, generator=gen),
        qzeros=torch.randint(-2 ** 31, 2 ** 31 - 1, (G, N // 8), dtype=torch.int32, device=dev, generator=gen),
        scales=(torch.rand((G, N), device=dev, generator=gen) * 0.015 + 0.005).half(),
        groupsize=gs, K=K, N=N, G=G)
    if act_order:
        perm = torch.randperm(K, device=dev, generator=gen)
        g_idx = torch.empty(K, dtype=torch.int32, device=dev)
        g_idx[perm] = (torch.arange(K, device=dev) // gs).to(torch.int32)
        lay["g_idx"] = g_idx
    else:
        lay["g_idx"] = None
    return lay


def time_graph(fn, steps, warmup):
    """Capture fn() once, replay `steps` times.  Returns (wall seconds, event seconds)."""
    import torch
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(max(warmup, 1)):
            fn()
    s.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        fn()
    with torch.cuda.stream(s):
        g.replay()
        s.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record(s)
        for _ in range(steps):
            g.replay()
        e1.record(s)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
    return t1 - t0, e0.elapsed_time(e1) * 1e-3


def bench_mlp_decode(M, steps, warmup, n_layers=32, seed=1, grouped=True):
    """One step = one token (M rows) through the MLP products of n_layers decoder layers over distinct weights:
    gate and up (which share their input) as ONE grouped launch on their own tensors, then down.
    grouped=False issues gate and up as two launches.  Returns the whole-step figures and, from two more graphs
    holding only the gate|up launches and only the down launches, the average duration of each kernel."""
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    gen = torch.Generator(device="cuda").manual_seed(seed)
    shapes = [("gate", 4096, 11008), ("up", 4096, 11008), ("down", 11008, 4096)]
    layers = [[make_layer_gpu(K, N, 128, gen) for _, K, N in shapes] for _ in range(n_layers)]
    x = torch.randn((M, 4096), device="cuda", generator=gen).half()
    h = torch.randn((M, 11008), device="cuda", generator=gen).half()
    outs = [torch.empty((M, 11008), dtype=torch.float16, device="cuda"),
            torch.empty((M, 11008), dtype=torch.float16, device="cuda"),
            torch.empty((M, 4096), dtype=torch.float16, device="cuda")]

    def gate_up(lay):
        if grouped:
            quant_hip.gemv_grouped(x, [(l["qweight"], l["qzeros"], l["scales"]) for l in lay[:2]], 128, outs=outs[:2])
        else:
            for l, out in zip(lay[:2], outs[:2]):
                quant_hip.gemv(x, l["qweight"], l["qzeros"], l["scales"], None, 128, out=out)

    def down(lay):
        l = lay[2]
        quant_hip.gemv(h, l["qweight"], l["qzeros"], l["scales"], None, 128, out=outs[2])

    def step():
        for lay in layers:
            gate_up(lay)
            down(lay)

    # sanity: the timed path computes the right thing (against the HIP dense dequant + fp32 matmul)
    errs = []
    gate_up(layers[0])
    down(layers[0])
    for l, inp, out in zip(layers[0], (x, x, h), outs):
        W = quant_hip.dequant(l["qweight"], l["qzeros"], l["scales"], None, 128)
        ref = inp.float() @ W.float()
        errs.append(float((out.float() - ref).abs().max() / ref.abs().max()))
        del W, ref
    err = max(errs)
    assert err < 1e-2, f"gemv sanity check failed: {errs}"

    wall, ev = time_graph(step, steps, warmup)
    _, ev_gu = time_graph(lambda: [gate_up(lay) for lay in layers], steps, 1)
    _, ev_dn = time_graph(lambda: [down(lay) for lay in layers], steps, 1)
    b_one = gemv_bytes(M, 4096, 11008, 32)                      # same total for the down shape
    b_gu = 2 * b_one - 2 * M * 4096 if grouped else b_one       # grouped: the shared activations are read once
    launches_gu = n_layers if grouped else 2 * n_layers
    launches = launches_gu + n_layers
    bytes_per_step = launches_gu * b_gu + n_layers * b_one
    us_gu = ev_gu / (steps * launches_gu) * 1e6
    us_dn = ev_dn / (steps * n_layers) * 1e6
    return dict(wall_s=wall, event_s=ev, steps=steps, launches_per_step=launches, bytes_per_step=bytes_per_step,
                gbs_wall=bytes_per_step * steps / wall / 1e9,
                gate_up=dict(bytes=b_gu, us=us_gu, gbs=b_gu / us_gu / 1e3),
                down=dict(bytes=b_one, us=us_dn, gbs=b_one / us_dn / 1e3),
                sum_of_kernels_ms=(launches_gu * us_gu + n_layers * us_dn) * 1e-3, sanity_rel_err=err)


def bench_single_gemv(K, N, M, act_order, reps, copies, seed=3):
    """One shape, `copies` distinct weight sets cycled (cold) -> GB/s from events."""
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    gen = torch.Generator(device="cuda").manual_seed(seed)
    lays = [make_layer_gpu(K, N, 128, gen, act_order) for _ in range(copies)]
    x = torch.randn((M, K), device="cuda", generator=gen).half()
    out = torch.empty((M, N), dtype=torch.float16, device="cuda")

    inner = max(1, 24 // copies)          # keep >= 24 launches per graph replay so the replay cost is amortised

    def step():
        for _ in range(inner):
            for l in lays:
                quant_hip.gemv(x, l["qweight"], l["qzeros"], l["scales"], l["g_idx"], 128, out=out)
    _, ev = time_graph(step, reps, 2)
    per = ev / (reps * copies * inner)
    b = gemv_bytes(M, K, N, lays[0]["G"], act_order)
    return dict(us=per * 1e6, gbs=b / per / 1e9, frac_hbm=b / per / 1e9 / HBM_PEAK_GBS, bytes=b, copies=copies)


def bench_mlp_decode_one_launch(M, steps, n_layers=32, seed=1):
    """The headline step through quant_hip.mlp_decode: per layer ONE launch computes gate, up, silu(gate) * up and down
    (the same packed bytes as the grouped gate|up + down launches, plus the activation)."""
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    gen = torch.Generator(device="cuda").manual_seed(seed)
    shapes = [("gate", 4096, 11008), ("up", 4096, 11008), ("down", 11008, 4096)]
    layers = [[make_layer_gpu(K, N, 128, gen) for _, K, N in shapes] for _ in range(n_layers)]
    x = torch.randn((M, 4096), device="cuda", generator=gen).half()
    tup = lambda l: (l["qweight"], l["qzeros"], l["scales"])

    def step():
        for g, u, d in layers:
            quant_hip.mlp_decode(x, tup(g), tup(u), tup(d), 128)

    g, u, d = layers[0]
    y = quant_hip.mlp_decode(x, tup(g), tup(u), tup(d), 128)
    gg, uu = quant_hip.gemv_grouped(x, [tup(g), tup(u)], 128)
    ref = quant_hip.gemv(torch.nn.functional.silu(gg) * uu, *tup(d), None, 128)
    err = float((y.float() - ref.float()).abs().max() / ref.float().abs().max())
    assert err < 1e-2 and not quant_hip.mlp_decode_gave_up(), f"one-launch MLP sanity check failed: {err}"
    wall, ev = time_graph(step, steps, 2)
    assert not quant_hip.mlp_decode_gave_up()
    b = 3 * gemv_bytes(M, 4096, 11008, 32) - 2 * M * 4096
    per = ev / (steps * n_layers)
    return dict(us_per_mlp=per * 1e6, step_gbs=b * n_layers / (wall / steps) / 1e9, kernel_gbs=b / per / 1e9,
                frac_hbm=b / per / 1e9 / HBM_PEAK_GBS, bytes_per_launch=b, launches_per_step=n_layers)


def bench_grouped_gemv(K, Ns, M, reps, copies, seed=4):
    """Several layers that share their input in one grouped launch (q|k|v of an attention block)."""
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    gen = torch.Generator(device="cuda").manual_seed(seed)
    sets = [[make_layer_gpu(K, N, 128, gen) for N in Ns] for _ in range(copies)]
    x = torch.randn((M, K), device="cuda", generator=gen).half()
    outs = [torch.empty((M, N), dtype=torch.float16, device="cuda") for N in Ns]
    inner = max(1, 24 // copies)

    def step():
        for _ in range(inner):
            for lays in sets:
                quant_hip.gemv_grouped(x, [(l["qweight"], l["qzeros"], l["scales"]) for l in lays], 128, outs=outs)
    _, ev = time_graph(step, reps, 2)
    per = ev / (reps * copies * inner)
    b = sum(gemv_bytes(M, K, N, K // 128) for N in Ns) - (len(Ns) - 1) * 2 * M * K
    return dict(us=per * 1e6, gbs=b / per / 1e9, frac_hbm=b / per / 1e9 / HBM_PEAK_GBS, bytes=b, copies=copies)


def bench_dequant(K, N, act_order, reps, copies=6, seed=9):
    """Dense dequantization (the reference's vecquant4recons_v2): bytes = packed layer read + fp16 matrix written."""
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    gen = torch.Generator(device="cuda").manual_seed(seed)
    lays = [make_layer_gpu(K, N, 128, gen, act_order) for _ in range(copies)]
    outs = [torch.empty((K, N), dtype=torch.float16, device="cuda") for _ in range(copies)]

    inner = 4                                # 24 launches per graph replay: the replay cost is amortised

    def step():
        for _ in range(inner):
            for l, o in zip(lays, outs):
                quant_hip.dequant(l["qweight"], l["qzeros"], l["scales"], l["g_idx"], 128, out=o)
    _, ev = time_graph(step, reps, 2)
    per = ev / (reps * copies * inner)
    G = lays[0]["G"]
    b = K * N // 2 + G * N // 2 + 2 * G * N + 4 * K + 2 * K * N
    return dict(us=per * 1e6, gbs=b / per / 1e9, frac_hbm=b / per / 1e9 / HBM_PEAK_GBS, bytes=b, copies=copies)


def bench_lora_step(reps, seed=5, dropout=0.0):
    """Config 2: Linear4bitLt 4096->4096, r=8, alpha=16, 2048 tokens: forward + backward
    (dx, dA, dB).  138.24 GFLOP of algorithmic work per step.  dropout > 0: the layer in training mode with that
    adapter dropout (the mask's seed is a launch argument, so that variant is timed eagerly only)."""
    import torch
    from alpaca_lora_4bit_amd import models
    gen = torch.Generator(device="cuda").manual_seed(seed)
    K = N = 4096
    M, r = 2048, 8
    lay = make_layer_gpu(K, N, 128, gen)
    m = models.Linear4bitLt("default", K, N, 128, False, r=r, lora_alpha=16, lora_dropout=dropout).cuda()
    m.qweight, m.qzeros, m.scales = lay["qweight"], lay["qzeros"], lay["scales"]
    m.g_idx = (torch.arange(K, device="cuda") // 128).to(torch.int32)
    m.bias = torch.zeros(N, dtype=torch.float16, device="cuda")
    m.train(dropout > 0)
    with torch.no_grad():
        m.lora_B["default"].weight.normal_(0, 0.02, generator=gen)
    x = torch.randn((8, 256, K), device="cuda", generator=gen).half().requires_grad_(True)
    dy = torch.randn((8, 256, N), device="cuda", generator=gen).half()

    def step():
        with torch.amp.autocast(device_type="cuda"):
            y = m(x)
        y.backward(dy)

    def clear():
        x.grad = None
        m.lora_A["default"].weight.grad = None
        m.lora_B["default"].weight.grad = None

    # eager: Python launches every kernel
    _spin_up(lambda: (step(), clear()))
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        step()
        clear()
    e1.record()
    torch.cuda.synchronize()
    eager = e0.elapsed_time(e1) * 1e-3 / reps
    flop = 2 * 2 * M * K * N + (2 * M * K * r + 2 * M * r * N) + 2 * (2 * M * K * r + 2 * M * r * N)
    if dropout > 0:
        return dict(eager_ms=eager * 1e3, eager_tokens_per_s=M / eager, eager_tflops=flop / eager / 1e12,
                    eager_frac_mfma=flop / eager / 1e12 / MFMA_FP16_PEAK_TFLOPS, dropout=dropout)

    # the same forward + backward captured once as a HIP graph and replayed (no Python between kernels)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(2):
            step()
            clear()
    s.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        step()
    with torch.cuda.stream(s):
        _spin_up(g.replay)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(s)
        for _ in range(reps):
            g.replay()
        e1.record(s)
        torch.cuda.synchronize()
    per = e0.elapsed_time(e1) * 1e-3 / reps
    return dict(ms=per * 1e3, tokens_per_s=M / per, tflops=flop / per / 1e12,
                frac_mfma=flop / per / 1e12 / MFMA_FP16_PEAK_TFLOPS, gflop_per_step=flop / 1e9,
                eager_ms=eager * 1e3, eager_tokens_per_s=M / eager)


def _random_llama7b(gen, n_layers=32):
    """Random-init LLaMA-7B decoder whose q/k/v/o/gate/up/down projections are 4-bit GPTQ layers (groupsize 128),
    fp16 everywhere else."""
    import torch
    from transformers import LlamaConfig, LlamaForCausalLM
    from alpaca_lora_4bit_amd import autograd_4bit as ag
    config = LlamaConfig(vocab_size=32000, hidden_size=4096, intermediate_size=11008, num_hidden_layers=n_layers,
                         num_attention_heads=32, num_key_value_heads=32, max_position_embeddings=2048,
                         tie_word_embeddings=False)
    with torch.device("meta"):
        model = LlamaForCausalLM(config)
    layers = ag.find_layers(model)
    layers.pop("lm_head", None)
    ag.make_quant_for_4bit_autograd(model, layers, groupsize=128)
    model = model.to_empty(device="cuda")
    with torch.no_grad():
        for name, mod in model.named_modules():
            if isinstance(mod, ag.Autograd4bitQuantLinear):
                K, N = mod.in_features, mod.out_features
                lay = make_layer_gpu(K, N, 128, gen)
                mod.qweight, mod.qzeros = lay["qweight"], lay["qzeros"]
                # about unit gain per layer (W entries ~ 6.5 * scale): activations stay finite through 32 layers
                mod.scales = (lay["scales"].float() * (0.15 / K ** 0.5 / 0.0125)).half()
                mod.g_idx = (torch.arange(K, device="cuda") // 128).to(torch.int32)
                mod.bias = torch.zeros(N, dtype=torch.float16, device="cuda")
        for name, p_ in model.named_parameters():
            if p_.dim() >= 2:
                p_.normal_(0, 0.02, generator=gen)
            else:
                p_.fill_(1.0)
    with contextlib.redirect_stdout(sys.stderr):     # stdout carries the one JSON line only
        ag.model_to_half(model)
    head_dim = config.hidden_size // config.num_attention_heads
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, head_dim, 2, device="cuda", dtype=torch.float32) / head_dim))
    for mod in model.modules():                      # rotary tables are plain buffers that to_empty left blank
        if hasattr(mod, "inv_freq"):
            mod.inv_freq = inv_freq.clone()
            if hasattr(mod, "original_inv_freq"):
                mod.original_inv_freq = inv_freq.clone()
    return model


def bench_llama7b_decode(new_tokens=64, prompt=16, seed=13):
    """Greedy generation with the random-init 4-bit LLaMA-7B through transformers' own `generate` (eager PyTorch,
    KV cache on), batch 1: tokens/s as the reference's inference.py prints it, first with one launch per projection,
    then with q+k+v and gate+up fused (model_attn_mlp_patch.make_quant_attn / make_fused_mlp), then with the token
    step replayed as a HIP graph (prefill, capture and replays all inside the timed region)."""
    import torch
    from alpaca_lora_4bit_amd.model_attn_mlp_patch import make_fused_mlp, make_quant_attn
    gen = torch.Generator(device="cuda").manual_seed(seed)
    model = _random_llama7b(gen)
    model.eval()
    ids = torch.randint(0, 32000, (1, prompt), device="cuda", generator=gen)

    def run():
        with torch.no_grad():
            model.generate(input_ids=ids, max_new_tokens=8, min_new_tokens=8, do_sample=False)       # warm-up
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            out = model.generate(input_ids=ids, max_new_tokens=new_tokens, min_new_tokens=new_tokens, do_sample=False)
            torch.cuda.synchronize()
        assert out.shape[1] == prompt + new_tokens
        return new_tokens / (time.perf_counter() - t0)

    res = {"new_tokens": new_tokens, "prompt": prompt, "tokens_per_s": run()}
    make_quant_attn(model)
    make_fused_mlp(model)
    res["tokens_per_s_fused_qkv_gate_up"] = run()
    # the same greedy decode with the one-token step replayed as a HIP graph (inference.greedy_generate_graph)
    from alpaca_lora_4bit_amd.inference import greedy_generate_graph
    greedy_generate_graph(model, ids, 8)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    out = greedy_generate_graph(model, ids, new_tokens)
    torch.cuda.synchronize()
    assert out.shape[1] == prompt + new_tokens
    res["tokens_per_s_fused_hip_graph"] = new_tokens / (time.perf_counter() - t0)
    del model
    torch.cuda.empty_cache()
    return res


def bench_llama7b_lora_train_step(reps=4, seed=11, n_layers=32, batch=4, seq=256, grouped=True):
    """configs[4] of the benchmark definition: random-init 32-layer LLaMA-7B decoder, every q/k/v/o/gate/up/down projection a 4-bit
    GPTQ layer (groupsize 128), LoRA r=8 alpha=16 on q_proj / v_proj, one forward + backward + AdamW step on
    batch 4 x seq 256 random token ids under fp16 autocast, gradient checkpointing off.  Eager PyTorch around
    the HIP kernels (attention = torch SDPA, lm_head = library GEMM).  grouped: q|k|v and gate|up of every block
    grouped in place (model_attn_mlp_patch.make_quant_attn / make_fused_mlp): one forward and one grad-input launch
    per group, on the layers' own tensors."""
    import torch
    from alpaca_lora_4bit_amd import autograd_4bit as ag
    from alpaca_lora_4bit_amd.models import inject_lora_layers
    gen = torch.Generator(device="cuda").manual_seed(seed)
    model = _random_llama7b(gen, n_layers)
    lora = inject_lora_layers(model, target_modules=("q_proj", "v_proj"), r=8, lora_alpha=16)
    if grouped:
        from alpaca_lora_4bit_amd.model_attn_mlp_patch import make_fused_mlp, make_quant_attn
        make_quant_attn(model)
        make_fused_mlp(model)
    with torch.no_grad():
        for l in lora.values():
            l.lora_B["default"].weight.normal_(0, 0.02, generator=gen)
    params = [p_ for p_ in model.parameters() if p_.requires_grad]
    opt = torch.optim.AdamW(params, lr=1e-4)
    ids = torch.randint(0, 32000, (batch, seq), device="cuda", generator=gen)
    model.train()
    model.config.use_cache = False

    def step():
        opt.zero_grad(set_to_none=True)
        with torch.amp.autocast(device_type="cuda", dtype=torch.float16):
            loss = model(input_ids=ids, labels=ids).loss
        (loss * 1024.0).backward()
        opt.step()
        return loss

    for _ in range(2):
        loss = step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        loss = step()
    e1.record()
    torch.cuda.synchronize()
    per = e0.elapsed_time(e1) * 1e-3 / reps
    tokens = batch * seq
    n_quant = sum(m.in_features * m.out_features for m in model.modules() if isinstance(m, ag.Autograd4bitQuantLinear))
    flop = 2 * 2 * tokens * n_quant                  # forward + grad-input products of the 4-bit layers
    out = dict(ms_per_step=per * 1e3, tokens_per_s=tokens / per, loss=float(loss.detach()), lora_layers=len(lora),
               quant_params=n_quant, tflops_4bit_layers=flop / per / 1e12,
               frac_mfma_4bit_layers=flop / per / 1e12 / MFMA_FP16_PEAK_TFLOPS,
               gpu_mem_gb=torch.cuda.max_memory_allocated() / 1e9)
    del model, opt, params, lora
    torch.cuda.empty_cache()
    return out


def _spin_up(fn, seconds=0.05):
    """Runs fn() back to back for about `seconds` of GPU time: after an idle gap (allocation, host work) the
    clocks need tens of milliseconds of load to come up, and a short timing loop would read 5-15 % slow."""
    import torch
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(8):
            fn()
        torch.cuda.synchronize()


def bench_gemm_only(M, K, N, act_order, reps, seed=7):
    import torch
    from alpaca_lora_4bit_amd import quant_hip
    gen = torch.Generator(device="cuda").manual_seed(seed)
    lay = make_layer_gpu(K, N, 128, gen, act_order)
    x = torch.randn((M, K), device="cuda", generator=gen).half()
    dy = torch.randn((M, N), device="cuda", generator=gen).half()
    res = {}
    for name, fn in (("fwd", lambda: quant_hip.gemm_fwd(x, lay["qweight"], lay["qzeros"], lay["scales"], lay["g_idx"], 128)),
                     ("bwd_dx", lambda: quant_hip.gemm_bwd_dx(dy, lay["qweight"], lay["qzeros"], lay["scales"], lay["g_idx"], 128))):
        _spin_up(fn)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        per = e0.elapsed_time(e1) * 1e-3 / reps
        res[name] = dict(us=per * 1e6, tflops=2 * M * K * N / per / 1e12,
                         frac_mfma=2 * M * K * N / per / 1e12 / MFMA_FP16_PEAK_TFLOPS)
    return res


def bench_mid_rows(reps):
    """Forward and grad-input products at 128 and 256 rows, 4096 x 4096 and the MLP shapes."""
    mid = {}
    for (M, K, N) in ((128, 4096, 4096), (256, 4096, 4096), (256, 4096, 11008), (256, 11008, 4096)):
        r = bench_gemm_only(M, K, N, False, reps)
        mid[f"M{M}_K{K}_N{N}"] = {"fwd_us": round(r["fwd"]["us"], 2), "bwd_dx_us": round(r["bwd_dx"]["us"], 2)}
    return mid


def cpu_baseline(seconds_budget=12.0):
    """Torch-CPU restatement of the reference's recons+matmul on the same workload shapes
    (one MLP: gate, up, down at M=1), repeated until ~seconds_budget of CPU time is spent."""
    import torch
    from oracle import q4_torch
    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    gen = torch.Generator().manual_seed(11)
    total_bytes, total_t, n = 0, 0.0, 0
    shapes = [(4096, 11008), (4096, 11008), (11008, 4096)]
    lays = []
    for K, N in shapes:
        G = K // 128
        lays.append(dict(
            qweight=torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 8, N), dtype=torch.int32, generator=gen),
            qzeros=torch.randint(-2 ** 31, 2 ** 31 - 1, (G, N // 8), dtype=torch.int32, generator=gen),
            scales=(torch.rand((G, N), generator=gen) * 0.015 + 0.005).half(),
            g_idx=(torch.arange(K) // 128).to(torch.int32),
            x=torch.randn((1, K), generator=gen).half(), K=K, N=N, G=G))
    q4_torch.matmul_recons(lays[0]["x"], lays[0]["qweight"], lays[0]["qzeros"], lays[0]["scales"], lays[0]["g_idx"])
    t_deq = 0.0                               # the dequantization part of it, timed inside the same calls
    while total_t < seconds_budget and n < 3000:
        for l in lays:
            t0 = time.perf_counter()
            W = q4_torch.dequant_v2(l["qweight"], l["qzeros"], l["scales"], l["g_idx"]).float()
            t1 = time.perf_counter()
            _ = l["x"].float() @ W
            t2 = time.perf_counter()
            t_deq += t1 - t0
            total_t += t2 - t0
            total_bytes += gemv_bytes(1, l["K"], l["N"], l["G"])
            n += 1
    return dict(value=total_bytes / total_t / 1e9, unit="GB/s", cores=cores, kind="port",
                sample=f"{n} GEMVs (gate/up/down of one MLP, M=1) through oracle/q4_torch.py "
                       f"(dense dequant + torch.matmul), {total_t:.1f} s of CPU time",
                ms_per_gemv=total_t / n * 1e3, ms_dequant=t_deq / n * 1e3, ms_matmul=(total_t - t_deq) / n * 1e3)


def cpu_baseline_lora_step(seconds_budget=12.0):
    """Config 2 on the host, the reference's algorithm with plain torch: forward = dense dequantization +
    torch.matmul (matmul_utils_4bit.py:114-127) + the adapter terms (models.py:58-66); backward = dense dequantization
    again + dy @ W^T (autograd_4bit.py:45-54) + the adapter's share of dx and the gradients of A and B.
    M = 2048 tokens, K = N = 4096, r = 8, scaling 2.  One warm-up, then the median of at least 5 steps."""
    import torch
    from oracle import q4_torch
    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    gen = torch.Generator().manual_seed(12)
    M, K, N, r, scaling = 2048, 4096, 4096, 8, 2.0
    G = K // 128
    qweight = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 8, N), dtype=torch.int32, generator=gen)
    qzeros = torch.randint(-2 ** 31, 2 ** 31 - 1, (G, N // 8), dtype=torch.int32, generator=gen)
    scales = (torch.rand((G, N), generator=gen) * 0.015 + 0.005).half()
    g_idx = (torch.arange(K) // 128).to(torch.int32)
    x = torch.randn((M, K), generator=gen).half().float()
    dy = torch.randn((M, N), generator=gen).half().float()
    A = (torch.rand((r, K), generator=gen) * 2 - 1) * (1.0 / K) ** 0.5
    B = torch.randn((N, r), generator=gen) * 0.02
    times, t_deq, t_mm, t_lora = [], [], [], []
    t_start = time.perf_counter()
    while len(times) < 6 or (time.perf_counter() - t_start < seconds_budget and len(times) < 30):
        t0 = time.perf_counter()
        W = q4_torch.dequant_v2(qweight, qzeros, scales, g_idx).float()
        t1 = time.perf_counter()
        y = x @ W
        t2 = time.perf_counter()
        xa = x @ A.t()
        y += scaling * (xa @ B.t())
        t3 = time.perf_counter()
        W = q4_torch.dequant_v2(qweight, qzeros, scales, g_idx).float()        # the backward dequantizes again
        t4 = time.perf_counter()
        dx = dy @ W.t()
        t5 = time.perf_counter()
        dyb = dy @ B
        dx += scaling * (dyb @ A)
        dB = scaling * (dy.t() @ xa)
        dA = scaling * (dyb.t() @ x)
        t6 = time.perf_counter()
        times.append(t6 - t0)
        t_deq.append((t1 - t0) + (t4 - t3)); t_mm.append((t2 - t1) + (t5 - t4)); t_lora.append((t3 - t2) + (t6 - t5))
        del W, y, dx, dB, dA
    med = lambda v: sorted(v[1:])[len(v[1:]) // 2]
    step = med(times)
    return dict(tokens_per_s=M / step, ms_per_step=step * 1e3, ms_dequant=med(t_deq) * 1e3, ms_matmul=med(t_mm) * 1e3,
                ms_adapter=med(t_lora) * 1e3, cores=cores, steps_timed=len(times) - 1,
                sample="config 2 (M=2048, K=N=4096, r=8) forward + backward on the host: oracle/q4_torch.py dense dequant "
                       "(twice, as the reference's forward and backward do) + torch.matmul fp32 + adapter terms and gradients")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="headline workload only (for profiling runs)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy: a kernel of known traffic for scaling rocprofv3 "
                         "FETCH_SIZE / WRITE_SIZE counters")
    ap.add_argument("--llama7b-step-only", action="store_true",
                    help="run only the config-4 full-model LoRA training step (32-layer LLaMA-7B shapes, random init)")
    ap.add_argument("--ungrouped", action="store_true",
                    help="with --llama7b-step-only: every projection its own launch (no in-place grouping of q|k|v, gate|up)")
    ap.add_argument("--llama7b-decode-only", action="store_true",
                    help="run only the greedy decode of the random-init 4-bit LLaMA-7B through transformers' generate")
    ap.add_argument("--mlp-one-launch-only", action="store_true",
                    help="run only the headline step through the one-launch MLP kernel (short run for profiling)")
    ap.add_argument("--dequant-only", action="store_true",
                    help="run only the dense dequantization of a 4096x11008 layer (short run for profiling)")
    ap.add_argument("--mid-rows-only", action="store_true",
                    help="only the 128- and 256-row products (for profiling runs)")
    ap.add_argument("--lora-step-only", action="store_true",
                    help="run only the config-2 LoRA layer step (forward + backward, M=2048) and print its figures: "
                         "a short run for profiling the GEMM and adapter kernels")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU's share of the path only; --gpus must be 1 "
              "(no collective or multi-GPU code exists in this repository).", file=sys.stderr)
        sys.exit(2)

    import torch
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    from alpaca_lora_4bit_amd import quant_hip  # noqa: F401  (fails loudly if the HIP library is missing)

    if args.llama7b_decode_only:
        r = bench_llama7b_decode()
        print(json.dumps({"workload": "llama7b_greedy_decode_b1", **{k: (round(v, 2) if isinstance(v, float) else v) for k, v in r.items()}}))
        return
    if args.llama7b_step_only:
        r = bench_llama7b_lora_train_step(max(args.steps, 2), grouped=not args.ungrouped)
        print(json.dumps({"workload": "config4_llama7b_lora_train_step_b4_s256", "grouped": not args.ungrouped,
                          **{k: (round(v, 4) if isinstance(v, float) else v) for k, v in r.items()}}))
        return
    if args.mlp_one_launch_only:
        r = bench_mlp_decode_one_launch(1, max(args.steps, 5))
        print(json.dumps({"workload": "mlp_decode_M1_one_launch_per_layer", **{k: (round(v, 4) if isinstance(v, float) else v) for k, v in r.items()}}))
        return
    if args.dequant_only:
        r = bench_dequant(4096, 11008, False, max(args.steps, 5))
        print(json.dumps({"workload": "dense_dequant_K4096_N11008", **{k: (round(v, 4) if isinstance(v, float) else v) for k, v in r.items()}}))
        return
    if args.mid_rows_only:
        print(json.dumps({"workload": "gemm_some_hundred_rows", **bench_mid_rows(max(args.steps, 5))}))
        return
    if args.lora_step_only:
        r = bench_lora_step(max(args.steps, 5))
        rd = bench_lora_step(max(args.steps, 5), dropout=0.05)
        print(json.dumps({"workload": "config2_lora_fwd_bwd_M2048", **{k: round(v, 4) for k, v in r.items()},
                          "with_dropout_0.05": {k: round(v, 4) for k, v in rd.items()}}))
        return
    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    head = bench_mlp_decode(1, args.steps, args.warmup)
    out = {
        "metric": "4-bit GEMV HBM GB/s (%peak) at M=1; LoRA fwd+bwd tokens/sec, LLaMA-7B shapes",
        "value": round(head["gbs_wall"], 1),
        "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(head["wall_s"] / args.steps * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 (int4 weights, fp32 accumulate)", "data": "synthetic",
        "config": {"workload": "configs[1]: LLaMA-7B MLP decode GEMV, M=1, gate/up 4096->11008 + down 11008->4096, "
                               "groupsize 128, no act-order; step = 32 layers x (gate|up as one grouped launch on their "
                               "own tensors + down) over 2.25 GB of distinct packed weights, replayed as one HIP graph",
                   "M": 1, "layers": 32, "launches_per_step": head["launches_per_step"],
                   "bytes_per_step": head["bytes_per_step"]},
        "pct_of_hbm_peak": round(100 * head["gbs_wall"] / HBM_PEAK_GBS, 2),
        # dominant kernel = the grouped gate|up launch (two thirds of the step's bytes and most of its time)
        "roofline": {"bound": "hbm", "achieved": round(head["gate_up"]["gbs"], 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(head["gate_up"]["gbs"] / HBM_PEAK_GBS, 4), "traffic": GEMV_TRAFFIC_BYTES,
                     "traffic_source": GEMV_TRAFFIC_SOURCE,
                     "kernel": "q4::gemv_seq_group_kernel<4, 0> (gate|up, N = 2 x 11008)",
                     "bytes_per_launch": head["gate_up"]["bytes"], "avg_launch_us": round(head["gate_up"]["us"], 3),
                     "other_kernel": {"kernel": "q4::gemv_seq_kernel<4, 0, false> (down, 11008 -> 4096)",
                                      "bytes_per_launch": head["down"]["bytes"],
                                      "avg_launch_us": round(head["down"]["us"], 3),
                                      "frac": round(head["down"]["gbs"] / HBM_PEAK_GBS, 4)},
                     "sum_of_kernel_durations_ms": round(head["sum_of_kernels_ms"], 4)},
    }
    if not args.no_extra:
        extra = {}
        for M in (4, 16):
            r = bench_mlp_decode(M, max(args.steps // 2, 5), 2)
            extra[f"mlp_decode_M{M}"] = {"step_gbs": round(r["gbs_wall"], 1),
                                         "gate_up_grouped_us": round(r["gate_up"]["us"], 3),
                                         "gate_up_grouped_frac_hbm": round(r["gate_up"]["gbs"] / HBM_PEAK_GBS, 4),
                                         "down_us": round(r["down"]["us"], 3),
                                         "down_frac_hbm": round(r["down"]["gbs"] / HBM_PEAK_GBS, 4)}
        r = bench_mlp_decode(1, max(args.steps // 2, 5), 2, grouped=False)
        extra["mlp_decode_M1_three_launches"] = {"step_gbs": round(r["gbs_wall"], 1), "gate_or_up_us": round(r["gate_up"]["us"], 3),
                                                 "gate_or_up_frac_hbm": round(r["gate_up"]["gbs"] / HBM_PEAK_GBS, 4),
                                                 "down_us": round(r["down"]["us"], 3)}
        for M in (1, 4):
            one = bench_mlp_decode_one_launch(M, max(args.steps // 2, 5))
            extra[f"mlp_decode_M{M}_one_launch_per_layer"] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in one.items()}
        qkv = bench_grouped_gemv(4096, (4096, 4096, 4096), 1, 10, 13)         # how the 4096 x 4096 layers run in a model
        extra["qkv_grouped_3x4096x4096_M1"] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in qkv.items()}
        # gate and up share x: concatenated along N they are one launch of twice the size
        gu = bench_single_gemv(4096, 22016, 1, False, 10, 16)
        extra["mlp_decode_M1_gate_up_fused_N22016"] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in gu.items()}
        hot = bench_single_gemv(4096, 11008, 1, False, 20, 1)     # the headline shape with its weights cache-resident
        extra["mlp_decode_M1_gate_proj_hot_cache"] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in hot.items()}
        c0 = bench_single_gemv(4096, 4096, 1, False, 20, 40)
        extra["config0_K4096_N4096_M1_cold"] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in c0.items()}
        c0h = bench_single_gemv(4096, 4096, 1, False, 20, 1)
        extra["config0_K4096_N4096_M1_hot_cache"] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in c0h.items()}
        for M in (1, 16):
            c3 = bench_single_gemv(5120, 13824, M, True, 10, 12)     # includes the gather of x through the row sort
            extra[f"config3_actorder_K5120_N13824_M{M}"] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in c3.items()}
        quant_hip.actorder_repack = False
        c3g = bench_single_gemv(5120, 13824, 1, True, 10, 12)
        extra["config3_actorder_K5120_N13824_M1_gather_kernel"] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in c3g.items()}
        quant_hip.actorder_repack = True
        for (K, N, act, name) in ((4096, 11008, False, "dense_dequant_K4096_N11008"),
                                  (5120, 13824, True, "dense_dequant_actorder_K5120_N13824")):
            dq = bench_dequant(K, N, act, 10)
            extra[name] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in dq.items()}
        lo = bench_lora_step(20)
        extra["config2_lora_fwd_bwd_M2048"] = {k: round(v, 4) for k, v in lo.items()}
        lod = bench_lora_step(20, dropout=0.05)          # the reference's default --lora_dropout, fused path
        extra["config2_lora_fwd_bwd_M2048_dropout0.05"] = {k: round(v, 4) for k, v in lod.items()}
        gm = bench_gemm_only(2048, 4096, 4096, False, 20)
        extra["config2_gemm_kernels"] = {k: {kk: round(vv, 4) for kk, vv in v.items()} for k, v in gm.items()}
        g3 = bench_gemm_only(512, 5120, 13824, True, 10)
        extra["config3_actorder_M512"] = {k: {kk: round(vv, 4) for kk, vv in v.items()} for k, v in g3.items()}
        # between the decode and the training shapes: 128 and 256 rows (a short prompt; the reference's default
        # micro-batch of one 256-token sample) on the 4096 x 4096 projections and the MLP shapes
        extra["gemm_some_hundred_rows"] = bench_mid_rows(20)
        try:
            with contextlib.redirect_stdout(sys.stderr):
                c4 = bench_llama7b_lora_train_step(4)
                c4u = bench_llama7b_lora_train_step(4, grouped=False)
            extra["config4_llama7b_lora_train_step_b4_s256"] = {k: (round(v, 4) if isinstance(v, float) else v)
                                                                  for k, v in c4.items()}
            extra["config4_llama7b_lora_train_step_b4_s256"]["projections"] = "q|k|v and gate|up grouped in place"
            extra["config4_llama7b_lora_train_step_b4_s256"]["ms_per_step_every_projection_its_own_launch"] = round(c4u["ms_per_step"], 4)
        except Exception as e:                       # the headline line must not depend on the installed transformers
            extra["config4_llama7b_lora_train_step_b4_s256"] = {"error": f"{type(e).__name__}: {e}"[:300]}
        try:
            with contextlib.redirect_stdout(sys.stderr):
                dec = bench_llama7b_decode()
            extra["llama7b_greedy_decode_b1"] = {k: (round(v, 2) if isinstance(v, float) else v) for k, v in dec.items()}
        except Exception as e:
            extra["llama7b_greedy_decode_b1"] = {"error": f"{type(e).__name__}: {e}"[:300]}
        out["extra"] = extra
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
        out["cpu_baseline"]["value"] = round(out["cpu_baseline"]["value"], 4)
        for k in ("ms_per_gemv", "ms_dequant", "ms_matmul"):
            out["cpu_baseline"][k] = round(out["cpu_baseline"][k], 2)
        # the second half of the metric (LoRA fwd+bwd tokens/s) on the same host cores
        lo_cpu = cpu_baseline_lora_step()
        out["cpu_baseline"]["lora_fwd_bwd_M2048"] = {k: (round(v, 2) if isinstance(v, float) else v) for k, v in lo_cpu.items()}
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
