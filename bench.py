#!/usr/bin/env python
"""Headline benchmark: fwd + bwd + SGD step of the 10-layer RTP transformer LM (README configuration of
the reference: vocab 10240, ninp 2048, nhid 2048, 32 heads, 10 decoder layers, seq 32, batch 32) on ONE
MI355X, bf16 weights with fp32 master, 8 rotation shards emulated on the device, synthetic token ids.

    python bench.py --gpus 1 --steps K --warmup W

Prints one JSON line.  `value` is tokens/s over K timed steps with inputs resident in HBM.  `roofline`
is the dominant kernel of the step (the GEMM variant with the largest summed duration), timed per launch in
the timed mode itself: the step is captured once more with every GEMM launch carrying a device time-stamp
slot and replayed after the timed region (so the stamps do not perturb `value`).  `kernels` lists every
kernel of the library timed with HIP events on two further eager steps.  `cpu_baseline` is the CPU oracle
(stock torch layers, fp32) timed on this box's host cores.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

CFG = dict(vocab=10240, ninp=2048, nhid=2048, nhead=32, layers=10, seq=32, batch=32, shards=8)
PEAK = {"bf16_mfma_tflops": 2500.0, "fp32_mfma_tflops": 157.3, "hbm_gbs": 8000.0}
PROFILES = os.path.join(ROOT, "profiles")


def _variant_of(kernel: str):
    """Library name of a product kernel (gemm_bf16_128x64_kc_rc ...) from the symbol rocprofv3 prints for
    rtp::gemm_dma_kernel<T, BM, BN, A k-contiguous, B k-contiguous, ...>; None for anything else."""
    import re
    m = re.search(r"gemm_dma_kernelI(DF16b|f)Li(\d+)ELi(\d+)ELb([01])ELb([01])E", kernel)
    if not m:
        return None
    return "gemm_%s_%sx%s_%s_%s" % ("bf16" if m.group(1) == "DF16b" else "f32", m.group(2), m.group(3),
                                    "kc" if m.group(4) == "1" else "rc", "kc" if m.group(5) == "1" else "rc")


def _table_rows(path):
    """(header comment lines, {variant: last-column-by-name dict}) of one summary under profiles/: a '#' header, one line
    of column names, then one row per kernel whose numeric columns are the trailing fields."""
    head, cols, rows = [], None, {}
    with open(path) as f:
        for line in f:
            if line.startswith("#"):
                head.append(line[1:].strip())
                continue
            fields = line.split()
            if cols is None:
                cols = fields[1:]
                continue
            v = _variant_of(line)
            if v is None or len(fields) < len(cols) + 1:
                continue
            try:
                rows[v] = dict(zip(cols, (float(x) for x in fields[-len(cols):])))
            except ValueError:
                continue
    return head, rows


def profile_reference(variant: str) -> dict:
    """What the committed rocprofv3 summaries of this script's LM step say about one product variant: memory-side
    traffic per dispatch (FETCH_SIZE / WRITE_SIZE runs, already scaled by the copy-kernel factors stated in the file),
    rocprofv3's average dispatch duration, and the kernel's own execution span that this script printed in that same
    profiled run (the `bench_json` header line).  Missing files or rows give None entries: nothing is assumed."""
    ref = {"traffic_bytes": None, "rocprof_avg_us": None, "execution_span_us": None, "dispatch_over_execution_span": None,
           "source": ["profiles/lm_step_pmc_fetch_write.txt", "profiles/lm_step_kernel_trace.txt"]}
    try:
        _, rows = _table_rows(os.path.join(PROFILES, "lm_step_pmc_fetch_write.txt"))
        if variant in rows and "traffic_KiB" in rows[variant]:
            ref["traffic_bytes"] = rows[variant]["traffic_KiB"] * 1024.0
    except OSError:
        pass
    try:
        head, rows = _table_rows(os.path.join(PROFILES, "lm_step_kernel_trace.txt"))
        if variant in rows and "avg_us" in rows[variant]:
            ref["rocprof_avg_us"] = rows[variant]["avg_us"]
        for line in head:
            if line.startswith("bench_json:"):
                span = json.loads(line[len("bench_json:"):]).get("execution_span_us", {}).get(variant)
                if span:
                    ref["execution_span_us"] = float(span)
        if ref["rocprof_avg_us"] and ref["execution_span_us"]:
            ref["dispatch_over_execution_span"] = ref["rocprof_avg_us"] / ref["execution_span_us"]
    except (OSError, ValueError):
        pass
    return ref


def step_flops(c):
    """Algorithmic flops of one fwd+bwd step: 3 x (2*T*matmul params + attention core)."""
    t = c["seq"] * c["batch"]
    per_layer = 4 * c["ninp"] * c["ninp"] + 2 * c["ninp"] * c["nhid"]
    matmul = c["layers"] * per_layer + c["ninp"] * c["vocab"]
    attn = c["layers"] * 4 * c["batch"] * c["nhead"] * c["seq"] * c["seq"] * (c["ninp"] // c["nhead"])
    return 3.0 * (2.0 * t * matmul + attn)


def build(c, device, dtype):
    import torch
    from rtp_amd.models.transformer_lm_rtp import TransformerLM
    from rtp_amd.module.collectives import ShardStore

    torch.manual_seed(0)
    lm = TransformerLM(c["vocab"], c["ninp"], c["nhead"], c["nhid"], 0.0, 0.1, c["layers"], c["shards"], 0,
                       device=device, dtype=dtype)
    with torch.no_grad():  # every rotated weight ~U(-0.1, 0.1), logits bias 0, LayerNorm gamma 1 / beta 0
        for m in lm.modules():
            st = getattr(m, "_store", None)
            if isinstance(st, ShardStore):
                st.home.uniform_(-0.1, 0.1)
        for sh in lm[-1].linear.linears:
            sh.bias.zero_()
    return lm


def cpu_baseline(c, steps=5, warmup=2):
    """The oracle LM on the host cores, evaluated the reference's way: every rotated layer a loop over its `shards`
    shards (per-shard F.linear / F.embedding / attention, outputs concatenated or summed), fp32, same shapes, same
    step (zero grads, fwd, CE, bwd, clip, SGD)."""
    import torch
    import torch.nn.functional as F
    from oracle import rtp_oracle as O

    torch.manual_seed(0)
    ref = O.TransformerLM(c["vocab"], c["ninp"], c["nhead"], c["nhid"], c["layers"], ws=c["shards"], shard_loop=True)
    with torch.no_grad():
        for n, p in ref.named_parameters():
            if "norm" not in n:
                p.uniform_(-0.1, 0.1)
    ids = torch.randint(0, c["vocab"], (c["seq"], c["batch"]))
    tgt = torch.randint(0, c["vocab"], (c["seq"], c["batch"]))

    def one():
        for p in ref.parameters():
            p.grad = None
        loss = F.cross_entropy(ref(ids).view(-1, c["vocab"]), tgt.view(-1))
        loss.backward()
        with torch.no_grad():
            for p in ref.parameters():
                p.add_(p.grad.clamp_(-0.05, 0.05), alpha=-1e-3)

    for _ in range(warmup):
        one()
    times = []
    for _ in range(steps):
        t0 = time.perf_counter()
        one()
        times.append(time.perf_counter() - t0)
    dt = sorted(times)[len(times) // 2]
    return {"value": c["seq"] * c["batch"] / dt, "unit": "tokens/s", "cores": torch.get_num_threads(),
            "kind": "port", "sample": f"median of {steps} full steps of the same configuration after {warmup} warm-ups, "
            f"fp32, every rotated layer looped over its {c['shards']} shards as the reference does ({dt * 1e3:.0f} ms/step, "
            f"os.cpu_count()={os.cpu_count()})"}


def _time_cpu(one, steps):
    """Median wall time of `one()` over `steps` calls after one warm-up call."""
    one()
    times = []
    for _ in range(steps):
        t0 = time.perf_counter()
        one()
        times.append(time.perf_counter() - t0)
    return sorted(times)[len(times) // 2]


def attainable_peaks(dev):
    """What this box's GPU actually delivers for the two kernel families the step is made of, measured here and now:
    a large bf16 product (4096^3, the same GEMM kernel, random operands) and a 1 GiB device-to-device copy (the
    library's shard-copy kernel; larger than the 256 MB memory-side cache, so it is served by HBM).  The roofline fractions in the report are against the published peaks; these give
    the second denominator."""
    import torch
    from rtp_amd import ops
    n = 4096
    gen = torch.Generator().manual_seed(1)
    a = torch.randn(n, n, generator=gen).to(torch.bfloat16).to(dev)
    b = torch.randn(n, n, generator=gen).to(torch.bfloat16).to(dev)
    c = torch.empty(n, n, dtype=torch.bfloat16, device=dev)

    def gemm():
        ops.gemm_raw(torch.bfloat16, a=a.data_ptr(), b=b.data_ptr(), c_out=c.data_ptr(), m=n, n=n, k=n, lda=n, ldb=n,
                     ldc=n, a_kcontig=True, b_kcontig=True)

    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)

    def timed(fn, iters):
        for _ in range(3):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / iters

    t_gemm = timed(gemm, 10)
    t_copy = timed(lambda: ops.shard_copy(dst, src), 5)
    out = {"gemm_bf16_4096_cubed_tflops": 2.0 * n ** 3 / t_gemm / 1e12,
           "device_copy_1GiB_gbs": 2.0 * src.numel() / t_copy / 1e9,
           "note": "same GEMM kernel / the shard-copy kernel, run alone on this GPU; copy counts bytes read + written"}
    del src, dst
    # Yardstick outside the product path: the vendor library (torch.matmul -> hipBLASLt) on the same random data,
    # for the large product and for the LM's per-layer shapes, beside this library's own time for each.
    yard = {}
    for (m_, n_, k_) in ((4096, 4096, 4096), (1024, 2048, 2048), (1024, 6144, 2048), (1024, 10240, 2048)):
        x = torch.randn(m_, k_, generator=gen).to(torch.bfloat16).to(dev)
        w = torch.randn(n_, k_, generator=gen).to(torch.bfloat16).to(dev)
        y = torch.empty(m_, n_, dtype=torch.bfloat16, device=dev)
        wt = w.t()
        t_lib = timed(lambda: ops.gemm_raw(torch.bfloat16, a=x.data_ptr(), b=w.data_ptr(), c_out=y.data_ptr(), m=m_, n=n_,
                                           k=k_, lda=k_, ldb=k_, ldc=n_, a_kcontig=True, b_kcontig=True), 20)
        t_ven = timed(lambda: torch.matmul(x, wt, out=y), 20)
        fl = 2.0 * m_ * n_ * k_
        yard[f"{m_}x{n_}x{k_}"] = {"this_library_us": t_lib * 1e6, "this_library_tflops": fl / t_lib / 1e12,
                                   "torch_matmul_us": t_ven * 1e6, "torch_matmul_tflops": fl / t_ven / 1e12}
    out["yardstick_torch_matmul_same_data"] = yard
    # What the matrix pipes sustain with nothing else in the way: a register-only MFMA loop on every SIMD, with
    # constant and with normally distributed operands.  The second is the practical ceiling of a bf16 product.
    import ctypes
    from rtp_amd import _lib
    rate = ctypes.c_double(0.0)
    probe = {}
    for name, mode in (("constant_operands", 0), ("random_operands", 1)):
        _lib.check(_lib.load().rtp_probe_mfma_rate(torch.cuda.current_stream().cuda_stream, mode, 20000, ctypes.byref(rate)))
        probe[name] = rate.value
    out["mfma_register_loop_tflops"] = probe
    return out


def gemm_workload(shape, operands, engine, steps, warmup):
    """One bf16 product, repeated: the measurement behind the GEMM ceiling figures.  Run it under
    `rocprofv3 --pmc GRBM_GUI_ACTIVE` for the sustained clock (busy cycles / duration) with zero-filled and with random
    operands, and with --engine torch for the vendor library's time on the same data."""
    import torch
    from rtp_amd import ops
    dev = torch.device("cuda", 0)
    m, n, k = (int(v) for v in shape.lower().split("x"))
    gen = torch.Generator().manual_seed(1)
    if operands == "random":
        x = torch.randn(m, k, generator=gen).to(torch.bfloat16).to(dev)
        w = torch.randn(n, k, generator=gen).to(torch.bfloat16).to(dev)
    else:
        x = torch.zeros(m, k, dtype=torch.bfloat16, device=dev)
        w = torch.zeros(n, k, dtype=torch.bfloat16, device=dev)
    y = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
    wt = w.t()
    if engine == "rtp":
        def one():
            ops.gemm_raw(torch.bfloat16, a=x.data_ptr(), b=w.data_ptr(), c_out=y.data_ptr(), m=m, n=n, k=k, lda=k, ldb=k,
                         ldc=n, a_kcontig=True, b_kcontig=True)
    else:
        def one():
            torch.matmul(x, wt, out=y)
    for _ in range(warmup):
        one()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(steps):
        one()
    e1.record()
    torch.cuda.synchronize()
    t = e0.elapsed_time(e1) * 1e-3 / steps
    print(json.dumps({"metric": "bf16 product, TFLOP/s", "value": 2.0 * m * n * k / t / 1e12, "unit": "TFLOP/s",
                      "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": t * 1e3, "higher_is_better": True,
                      "dtype": "bf16", "data": "synthetic",
                      "config": {"workload": f"one product {m}x{n}x{k}, {operands} operands, engine {engine}"}}))


def linear_ring_baseline():
    """BASELINE configuration 1 the way the reference runs it: two gloo ranks on the host cores, each with half of the
    batch rows and one home shard, the shards (and their gradients) travelling the ring.  The rank processes are
    started by this call, which must come before this process has touched the GPU."""
    import torch
    from oracle import gloo_ring
    gen = torch.Generator().manual_seed(0)
    w = torch.rand(2048, 2048, generator=gen) * 0.2 - 0.1
    x_cpu, g_cpu = torch.randn(1024, 2048, generator=gen), torch.randn(1024, 2048, generator=gen)
    threads = max(1, torch.get_num_threads() // 2)
    # gloo announces its connections on stdout, in the rank processes: for the duration of the ring, file descriptor
    # 1 (which they inherit) is stderr, so that this script's stdout stays the one JSON line
    sys.stdout.flush()
    saved = os.dup(1)
    os.dup2(2, 1)
    try:
        res = gloo_ring.column_linear_ring(x_cpu, w, torch.zeros(2048), g_cpu, ws=2, steps=5, warmup=2,
                                           threads_per_rank=threads)
    finally:
        sys.stdout.flush()
        os.dup2(saved, 1)
        os.close(saved)
    return (sorted(res["times"])[2], 2 * threads, "median of 5 fwd+bwd passes after 2 warm-ups, 2 gloo ranks on loopback")


def layer_workload(name, steps, warmup, graph=True, cpu=True, ring_result=None):
    """The reference's other configurations (single rotated layers), fwd+bwd, timed with the same event
    bracketing; returns the JSON record with the layer's own algorithmic work and the dominant kernel's roofline."""
    import torch
    import torch.nn as nn
    from rtp_amd import _lib, emulate_shards

    gen = torch.Generator().manual_seed(0)

    def uni(*shape):
        return torch.rand(*shape, generator=gen) * 0.2 - 0.1

    if name == "linear":
        master = nn.Linear(2048, 2048)
        with torch.no_grad():
            master.weight.copy_(uni(2048, 2048)), master.bias.zero_()
        x_cpu, g_cpu = torch.randn(1024, 2048, generator=gen), torch.randn(1024, 2048, generator=gen)
        if cpu and ring_result is None:
            ring_result = linear_ring_baseline()   # same seed, same draws: identical operands

    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    if name == "linear":  # fp32 column-parallel Linear [1024,2048] x [2048,2048], 2 shards
        from rtp_amd.module.linear import ColumnParallelLinear
        with emulate_shards(2):
            layer = ColumnParallelLinear(2048, 2048, linear_layer=master, device=dev, dtype=torch.float32)
        x = x_cpu.to(dev).requires_grad_()
        g = g_cpu.to(dev)
        fn = lambda: layer(x).backward(g)
        cpu_fn = lambda: ring_result
        work = {"flops": 3 * 2.0 * 1024 * 2048 * 2048, "bytes": None, "bound": "mfma", "peak": PEAK["fp32_mfma_tflops"],
                "dtype": "f32", "desc": "column-parallel Linear fwd+bwd, X [1024,2048], W [2048,2048], 2 shards, fp32"}
    elif name == "embedding":  # table [10240,2048] fp32, 4 shards, ids [32,32]
        from rtp_amd.module.embedding import ParallelEmbedding
        master = nn.Embedding(10240, 2048)
        with torch.no_grad():
            master.weight.copy_(uni(10240, 2048))
        layer = ParallelEmbedding(10240, 2048, 4, 0, Embedding_layer=master, device=dev, dtype=torch.float32)
        ids_cpu, g_cpu = torch.randint(0, 10240, (32, 32), generator=gen), torch.randn(32, 32, 2048, generator=gen)
        ids, g = ids_cpu.to(dev), g_cpu.to(dev)
        fn = lambda: layer(ids).backward(g)

        def cpu_fn():
            from oracle import rtp_oracle as O
            table = master.weight.detach().clone().requires_grad_()

            def one():
                table.grad = None
                O.parallel_embedding(ids_cpu, table, 4).backward(g_cpu)
            return _time_cpu(one, 5), torch.get_num_threads(), "median of 5 fwd+bwd passes after 1 warm-up"
        # gather 16 MiB + scatter-add <= 24 MiB of algorithmic traffic (the 80 MiB dense zero fill is not counted)
        work = {"flops": None, "bytes": (16 + 24) * 2.0 ** 20, "bound": "hbm", "peak": PEAK["hbm_gbs"], "dtype": "f32",
                "desc": "vocab-sharded Embedding fwd+bwd, table [10240,2048] fp32 in 4 shards, ids [32,32]"}
    elif name == "attention":  # d_model 2048, 32 heads in 8 groups, batch 8, seq 512, causal, bf16
        from rtp_amd.module.attention import ParallelMultiheadAttention
        mha = nn.MultiheadAttention(2048, 32, bias=True)
        with torch.no_grad():
            for p_ in mha.parameters():
                p_.copy_(uni(*p_.shape))
        layer = ParallelMultiheadAttention(2048, 32, 8, 0, MultiheadAttention_layer=mha.to(torch.bfloat16), device=dev,
                                           dtype=torch.bfloat16)
        x_cpu, g_cpu = torch.randn(512, 8, 2048, generator=gen), torch.randn(512, 8, 2048, generator=gen)
        x = x_cpu.to(dev, torch.bfloat16).requires_grad_()
        g = g_cpu.to(dev, torch.bfloat16)
        fn = lambda: layer(x, x, x, is_causal=True, need_weights=False)[0].backward(g)

        def cpu_fn():
            from oracle import rtp_oracle as O
            ps = [p_.detach().float().clone().requires_grad_() for p_ in
                  (mha.in_proj_weight, mha.in_proj_bias, mha.out_proj.weight, mha.out_proj.bias)]
            xc = x_cpu.clone().requires_grad_()
            mask = torch.triu(torch.full((512, 512), float("-inf")), diagonal=1)

            def one():
                for t in ps + [xc]:
                    t.grad = None
                O.parallel_multihead_attention(xc, *ps, 32, 8, mask=mask)[0].backward(g_cpu)
            return _time_cpu(one, 3), torch.get_num_threads(), "median of 3 fwd+bwd passes after 1 warm-up, fp32"
        proj = 2.0 * 4096 * 2048 * (6144 + 2048)
        core = 4.0 * 8 * 32 * 512 * 512 * 64
        work = {"flops": 3 * proj + 3.5 * core, "bytes": None, "bound": "mfma", "peak": PEAK["bf16_mfma_tflops"],
                "dtype": "bf16", "desc": "head-sharded attention fwd+bwd, d_model 2048, 32 heads in 8 groups, batch 8, "
                "seq 512, causal, bf16 (attention core counted in full, not halved for causality)"}
    elif name == "moe":  # 8 experts, top-2, d_model 2048, d_ff 8192, 4096 tokens, bf16
        from rtp_amd.models.transformer_lm_rtp import FeedForwardLayer_expert
        from rtp_amd.module.moe import WeightMOELayer
        from rtp_amd.module.top2gate import Top2Gate, WeightTop2Gate
        mg = Top2Gate(2048, 8)
        with torch.no_grad():
            mg.wg.weight.copy_(uni(8, 2048))
        masters = []
        for _ in range(8):
            m = FeedForwardLayer_expert(2048, 8192, nn.ReLU(), 0.0)
            with torch.no_grad():
                for p_ in m.parameters():
                    p_.copy_(uni(*p_.shape))
            masters.append(m.to(torch.bfloat16))
        with emulate_shards(8):
            gate = WeightTop2Gate(2048, 8, gate=mg.to(torch.bfloat16), device=dev, dtype=torch.bfloat16)
            local = nn.ModuleList([FeedForwardLayer_expert(2048, 8192, nn.ReLU(), 0.0)])
            layer = WeightMOELayer(gate, local, device=dev, dtype=torch.bfloat16,
                                   original_experts=[nn.ModuleList([m]) for m in masters])
        x_cpu, g_cpu = torch.randn(8, 512, 2048, generator=gen), torch.randn(8, 512, 2048, generator=gen)
        x = x_cpu.to(dev, torch.bfloat16).requires_grad_()
        g = g_cpu.to(dev, torch.bfloat16)
        u = torch.rand(4096, 8, generator=gen).clamp(min=torch.finfo(torch.float32).tiny, max=1 - torch.finfo(torch.float32).eps)
        noise_cpu = -torch.log(-torch.log(u))  # Gumbel(0,1) routing noise, drawn on the host
        noise = noise_cpu.to(dev)
        fn = lambda: layer(x, noise=noise).backward(g)

        def cpu_fn():
            from oracle import rtp_oracle as O
            wg = mg.wg.weight.detach().float().clone().requires_grad_()
            experts = [tuple(p_.detach().float().clone().requires_grad_() for p_ in m.parameters()) for m in masters]
            xc = x_cpu.clone().requires_grad_()

            def one():
                for t in [wg, xc] + [t for e in experts for t in e]:
                    t.grad = None
                (O.moe_layer(xc, wg, experts, noise_cpu, 8)[0] * g_cpu).sum().backward()
            return _time_cpu(one, 1), torch.get_num_threads(), "1 fwd+bwd pass after 1 warm-up, fp32, the " \
                "reference's dense dispatch / combine einsums"
        work = {"flops": 3 * 8192 * 2.0 * 2 * 2048 * 8192, "bytes": None, "bound": "mfma", "peak": PEAK["bf16_mfma_tflops"],
                "dtype": "bf16", "desc": "expert-sharded MoE layer fwd+bwd, 8 experts, top-2, d_model 2048, d_ff 8192, "
                "4096 tokens, bf16 (flops for 8192 routed pairs, i.e. nothing dropped)"}
    else:
        raise SystemExit(f"unknown workload {name}")

    from rtp_amd import ring
    from rtp_amd.module.collectives import ShardStore
    # Every pass starts like a training step, after zero_grad: the rotated gradients are overwritten, not added to
    # (what RotatedSGD.zero_grad arranges), and the input's gradient is a fresh tensor.
    stores = [m._store for m in layer.modules() if isinstance(getattr(m, "_store", None), ShardStore)]
    inputs = [] if name == "embedding" else [x]  # the embedding's input is token ids
    body = fn

    def fn():
        for st in stores:
            st.mark_overwrite()
        for t in inputs:
            t.grad = None
        body()

    # warm-up on a side stream, then the layer's forward + backward recorded once into a HIP graph and replayed
    # (as for the language-model step); --no-graph times eager launches, CPU launch overhead included
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(max(warmup, 1)):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    ring.fence(dev)
    run, launch_mode = fn, "eager (CPU launch overhead included)"
    if graph:
        cg = torch.cuda.CUDAGraph()
        with torch.cuda.graph(cg):
            fn()
        ring.fence(dev)
        run, launch_mode = cg.replay, "HIP graph replay"
        run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        run()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    _lib.profile_enable(True)
    fn(), fn()
    stats = _lib.profile_collect()
    _lib.profile_enable(False)
    kernels = {k: {"launches": v["launches"] // 2, "ms": round(v["total_ms"] / 2, 4),
                   "tflops": round(v["flops"] / max(v["total_ms"], 1e-9) / 1e9, 2),
                   "gbs": round(v["bytes"] / max(v["total_ms"], 1e-9) / 1e6, 1)} for k, v in sorted(stats.items())}
    # the dominant kernel: the one that takes the most time; for a memory-bound layer among the kernels that carry
    # its bytes (the id sort of the embedding backward takes the longest of its launches and moves 16 KB)
    heavy = {k: v for k, v in stats.items()
             if work["bound"] == "mfma" or v["bytes"] >= 0.05 * max(x["bytes"] for x in stats.values())}
    dom_name, dom = max(heavy.items(), key=lambda kv: kv[1]["total_ms"])
    avg_ms = dom["total_ms"] / dom["launches"]
    if work["bound"] == "mfma":
        achieved = dom["flops"] / dom["launches"] / (avg_ms * 1e-3) / 1e12
        whole = work["flops"] / dt / 1e12
        unit = "TFLOP/s"
    else:
        achieved = dom["bytes"] / dom["launches"] / (avg_ms * 1e-3) / 1e9
        whole = work["bytes"] / dt / 1e9
        unit = "GB/s"
    out = {"metric": f"fwd+bwd time of one rotated layer ({name})", "value": dt * 1e3, "unit": "ms", "n_gpus": 1,
           "steps": steps, "warmup": warmup, "ms_per_step": dt * 1e3, "higher_is_better": False, "scaling": "weak",
           "vs_baseline": None, "dtype": work["dtype"], "data": "synthetic",
           "config": {"workload": work["desc"], "launch_mode": launch_mode},
           "roofline": {"bound": work["bound"], "achieved": achieved, "peak": work["peak"], "unit": unit,
                        "frac": achieved / work["peak"], "traffic": None, "kernel": dom_name,
                        "avg_launch_us": avg_ms * 1e3},
           "whole_layer": {"achieved": whole, "unit": unit, "frac": whole / work["peak"]},
           "kernels": kernels}
    if cpu:
        # the CPU restatement of the same layer on this box's host cores: a reported baseline, not a target
        del layer
        torch.cuda.empty_cache()
        sec, cores, sample = cpu_fn()
        out["cpu_baseline"] = {"value": sec * 1e3, "unit": "ms", "cores": cores, "kind": "port",
                               "sample": f"{sample} (os.cpu_count()={os.cpu_count()})"}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--workload", default="lm", choices=["lm", "linear", "embedding", "attention", "moe", "gemm"],
                    help="lm: the headline training step (default); the others time one rotated layer of the "
                         "reference's remaining configurations, fwd+bwd")
    ap.add_argument("--sgd-overlap", dest="sgd_overlap", action="store_true",
                    help="apply each rotated layer's SGD update right after that layer's backward, on a second stream "
                         "(measured: no gain, the update and the backward compete for memory bandwidth)")
    ap.add_argument("--no-sgd-fused", dest="sgd_fused", action="store_false",
                    help="one clip + SGD launch over all parameters after the backward pass, instead of applying the "
                         "update of every weight matrix in the epilogue of its weight-gradient product (the default: "
                         "bit-identical weights, the gradients of those matrices are never written or read back)")
    ap.add_argument("--fused-head-loss", dest="fused_head_loss", action="store_true",
                    help="logits layer and cross-entropy as one operation whose [tokens, vocab] logits never reach "
                         "memory (statistics from the forward product's epilogue, the gradient from a second run of the "
                         "product); measured slower than writing the logits once at this token count, so not the default")
    ap.add_argument("--no-wgrad-overlap", dest="wgrad_overlap", action="store_false",
                    help="launch weight / bias gradient kernels on the compute stream instead of a second stream "
                         "beside the input-gradient chain")
    ap.add_argument("--optimizer", default="sgd", choices=["sgd", "adam"],
                    help="sgd: the headline configuration (default); adam: the reference harness's own optimiser "
                         "(clip 0.05, Adam lr 1e-3), fp32 moments beside the fp32 master")
    ap.add_argument("--rotation", default="direct", choices=["direct", "staged"],
                    help="direct (default): the products read every shard from its home row, the LDS stage ring of the "
                         "product kernel is the rotation's double buffer; staged: shards are first copied into two HBM "
                         "slots on a side stream (the transport of a multi-GPU ring)")
    ap.add_argument("--no-warm-ahead", dest="warm_ahead", action="store_false",
                    help="do not let a layer's first product request the next layer's shards, which brings them into "
                         "the memory-side cache before their own products run (direct rotation only)")
    ap.add_argument("--operands", default="random", choices=["random", "zeros"],
                    help="--workload gemm: normally distributed or all-zero bf16 operands")
    ap.add_argument("--engine", default="rtp", choices=["rtp", "torch"],
                    help="--workload gemm: this library's product kernel, or torch.matmul (the vendor library) as the "
                         "yardstick on the same data")
    ap.add_argument("--shape", default="4096x4096x4096", help="--workload gemm: MxNxK of y[M,N] = x[M,K] w[N,K]^T")
    ap.add_argument("--lm-only", action="store_true",
                    help="--workload lm: only the headline step (the default run then also times the same step under the "
                         "staged rotation and the reference's four single-layer configurations, after the timed region); "
                         "what the rocprofv3 summaries of the LM step are collected with, so that their per-kernel "
                         "averages hold the step's dispatches only")
    ap.add_argument("--no-graph", dest="graph", action="store_false",
                    help="launch every kernel eagerly instead of replaying the step from a captured HIP graph")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU's throughput: this build runs every rotation shard on a single MI355X and "
              f"has no multi-GPU path (--gpus {args.gpus} is not supported)", file=sys.stderr)
        sys.exit(2)

    if args.workload == "gemm":
        gemm_workload(args.shape, args.operands, args.engine, args.steps, args.warmup)
        return
    if args.workload != "lm":
        print(json.dumps(layer_workload(args.workload, args.steps, args.warmup, args.graph, not args.no_cpu_baseline)))
        return
    whole = not args.lm_only
    # the gloo ranks of configuration 1's CPU baseline are started before this process touches the GPU
    ring_result = linear_ring_baseline() if whole and not args.no_cpu_baseline else None

    import torch
    import torch.nn.functional as F
    from rtp_amd import _lib, ring, rotated_weight_bytes, staging_bytes
    from rtp_amd.module.loss import cross_entropy, linear_cross_entropy
    from rtp_amd.optim import RotatedAdam, RotatedSGD

    dev = torch.device("cuda", 0)
    ring.set_wgrad_overlap(args.wgrad_overlap)
    ring.set_rotation_mode(args.rotation)
    ring.set_warm_ahead(args.warm_ahead and args.rotation == "direct")
    torch.cuda.set_device(dev)
    c = CFG
    lm = build(c, dev, torch.bfloat16)
    if args.optimizer == "adam":
        opt = RotatedAdam(lm, lr=1e-3, clip_value=0.05)
    else:
        opt = RotatedSGD(lm, lr=1e-3, clip_value=0.05, overlap_backward=args.sgd_overlap,
                         fused_backward=args.sgd_fused and not args.sgd_overlap)
    gen = torch.Generator().manual_seed(0)
    # A fresh batch every step, as in the reference's loop (benchmarks/rtp_benchmark.py:149-186 draws one per
    # iteration): a pool of batches resident in HBM, and one 16 KiB device copy per step, inside the timed region,
    # into the buffer the (replayed) step reads its ids and targets from.
    pool = torch.randint(0, c["vocab"], (8, 2, c["seq"], c["batch"]), generator=gen).to(dev)
    batch = pool[0].clone()
    ids, tgt = batch[0], batch[1]
    tokens = c["seq"] * c["batch"]
    loss_box = [None]

    def step():
        opt.zero_grad()
        if args.fused_head_loss:
            hidden = ids
            for layer in list(lm)[:-1]:
                hidden = layer(hidden)
            loss = linear_cross_entropy(hidden, lm[-1].linear, tgt.view(-1))
        else:
            logits = lm(ids)
            loss = cross_entropy(logits.view(-1, c["vocab"]), tgt.view(-1))
        loss.backward()
        opt.step()
        loss_box[0] = loss.detach()  # detached: a live autograd graph would pin last step's AccumulateGrad nodes

    def timed(n_warm, n_steps):
        """(seconds per step, the replayed graph or None): warm-up on a side stream (the documented recipe for
        whole-step graph capture: autograd's gradient accumulators remember the stream they were created on, and it
        must not be the default stream), the whole step -- both streams of the rotation included -- recorded once into a
        HIP graph, then n_steps replays bracketed by device synchronisations."""
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(max(n_warm, 1)):
                step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        ring.fence(dev)
        first = float(loss_box[0])
        run, g = step, None
        if args.graph:
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                step()
            ring.fence(dev)  # the ring's last fence was recorded inside the capture; re-arm it for eager use
            run = g.replay
            run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(n_steps):
            batch.copy_(pool[(i + 1) % pool.shape[0]])
            run()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n_steps, g, first

    dt, g, first_loss = timed(args.warmup, args.steps)
    last_loss = float(loss_box[0])

    # The dominant kernel in the TIMED mode (graph replay, both streams live): the step is captured a second time
    # with the GEMM launches carrying device time-stamp slots (HIP timing events do not work inside a replayed
    # graph), replayed, and the per-launch durations read back after every replay.
    graph_stats, instr_ms = None, None
    if args.graph:
        _lib.profile_enable(2)
        g2 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g2):
            step()
        ring.fence(dev)
        _lib.profile_enable(0)
        stream = torch.cuda.current_stream().cuda_stream
        g2.replay()
        torch.cuda.synchronize()
        reps, graph_stats = 5, {}
        t_i = 0.0
        for _ in range(reps):
            _lib.profile_reset_stamps(stream)
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            g2.replay()
            torch.cuda.synchronize()
            t_i += time.perf_counter() - t1
            for k, v in _lib.profile_collect(clear=False).items():
                acc = graph_stats.setdefault(k, {"launches": 0, "total_ms": 0.0, "flops": 0.0, "bytes": 0.0,
                                                 "phase_ms": [0.0] * 4})
                for f in ("launches", "total_ms", "flops", "bytes"):
                    acc[f] += v[f]
                acc["phase_ms"] = [a + b for a, b in zip(acc["phase_ms"], v["phase_ms"])]
        instr_ms = t_i / reps * 1e3
        _lib.profile_collect()
        del g2

    # Per-kernel timing with HIP events around every launch in extra EAGER steps: every kernel of the library, for the
    # `kernels` table.  With an event pair per launch the host cannot keep the GPU fed (eager_ms_per_step below), so
    # the two streams hardly overlap here: these are not the timed mode's durations.
    _lib.profile_enable(True)
    prof_steps = 2
    torch.cuda.synchronize()
    t_e = time.perf_counter()
    for _ in range(prof_steps):
        step()
    torch.cuda.synchronize()
    eager_ms = (time.perf_counter() - t_e) / prof_steps * 1e3
    stats = _lib.profile_collect()
    _lib.profile_enable(False)
    gemms = {k: v for k, v in stats.items() if k.startswith("gemm_")}
    timed_gemms = {k: v for k, v in (graph_stats or stats).items() if k.startswith("gemm_")}
    dom_name, dom = max(timed_gemms.items(), key=lambda kv: kv[1]["total_ms"])
    span_us = dom["total_ms"] / dom["launches"] * 1e3
    # rocprofv3 reports a longer duration for the same dispatches than the kernel's own first-wave-to-last-wave span:
    # its clock starts when the queue reaches the dispatch, and the workgroups then still wait for the CUs that the
    # other stream's product holds.  The ratio of the two is read from the committed rocprofv3 summary of this very
    # command (profiles/lm_step_kernel_trace.txt: the kernel's average duration / the span this script printed in
    # that run); the roofline figure is quoted on the longer, rocprofv3-compatible span.
    prof_ref = profile_reference(dom_name)
    ratio = (prof_ref["dispatch_over_execution_span"] or 1.0) if graph_stats is not None else 1.0
    avg_ms = span_us * ratio * 1e-3
    achieved = dom["flops"] / dom["launches"] / (avg_ms * 1e-3) / 1e12
    # Which roof bounds the kernel: the larger of its two minimum times, flops at the MFMA peak or algorithmic bytes
    # at the HBM peak.  A weight-gradient product that carries the optimiser's update moves 10 bytes per output
    # element on top of its operands, against 2 * K flops with K = the step's 1024 tokens: ~125 flop per byte, below
    # the machine's 312, so its roof is the memory system's; the other products are bound by the matrix pipes.
    alg_bytes = dom["bytes"] / dom["launches"]
    mfma_frac = achieved / PEAK["bf16_mfma_tflops"]
    hbm_gbs = alg_bytes / (avg_ms * 1e-3) / 1e9
    hbm_frac = hbm_gbs / PEAK["hbm_gbs"]
    if hbm_frac > mfma_frac:
        roof = {"bound": "hbm", "achieved": hbm_gbs, "peak": PEAK["hbm_gbs"], "unit": "GB/s", "frac": hbm_frac,
                "mfma_view": {"achieved": achieved, "peak": PEAK["bf16_mfma_tflops"], "unit": "TFLOP/s", "frac": mfma_frac}}
    else:
        roof = {"bound": "mfma", "achieved": achieved, "peak": PEAK["bf16_mfma_tflops"], "unit": "TFLOP/s",
                "frac": mfma_frac,
                "hbm_view": {"achieved": hbm_gbs, "peak": PEAK["hbm_gbs"], "unit": "GB/s", "frac": hbm_frac}}
    span = {"avg_launch_us": span_us, "frac": (hbm_frac if hbm_frac > mfma_frac else mfma_frac) * avg_ms * 1e3 / span_us,
            "what": "first wave's start to last wave's end of the kernel (device time stamps in the replayed HIP graph; HIP "
                    "events in eager mode): its own execution, without the wait for CUs that a dispatch span includes",
            "instrumented_replay_ms_per_step": instr_ms}
    all_gemm_ms = sum(v["total_ms"] for v in gemms.values()) / prof_steps
    all_gemm_tflops = sum(v["flops"] for v in gemms.values()) / prof_steps / (all_gemm_ms * 1e-3) / 1e12
    copy = stats.get("shard_copy")
    kernels = {k: {"launches_per_step": v["launches"] // prof_steps, "ms_per_step": round(v["total_ms"] / prof_steps, 4),
                   "tflops": round(v["flops"] / max(v["total_ms"], 1e-9) / 1e9, 2),
                   "gbs": round(v["bytes"] / max(v["total_ms"], 1e-9) / 1e6, 1)} for k, v in sorted(stats.items())}
    graph_gemms = None if graph_stats is None else {
        k: {"launches_per_step": v["launches"] // 5, "avg_launch_us": round(v["total_ms"] / v["launches"] * 1e3, 3),
            "tflops": round(v["flops"] / max(v["total_ms"], 1e-9) / 1e9, 2),
            # a workgroup's time, averaged over the workgroups of a launch and over the launches: waiting for a CU after
            # the launch's first workgroup started, entry -> first operands in LDS, the K loop, the epilogue
            "workgroup_phases_us": dict(zip(("wait_for_cu", "to_first_slab", "k_loop", "epilogue"),
                                            (round(x / v["launches"] * 1e3, 2) for x in v["phase_ms"])))}
        for k, v in sorted(graph_stats.items())}

    flops = step_flops(c)
    peaks = attainable_peaks(dev)
    out = {
        "metric": "fwd+bwd tokens/s, 10-layer RTP LM, 1 MI355X; % MFMA peak; peak weight bytes",
        "value": tokens / dt, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"10-layer RTP transformer LM fwd+bwd+{args.optimizer.upper()} step: vocab 10240, ninp 2048, nhid 2048, "
                               "32 heads, seq 32, batch 32, bf16 weights + fp32 master, 8 rotation shards emulated on "
                               "one GPU, a fresh batch of uniform random token ids every step, weights U(-0.1,0.1), dropout 0, lr 1e-3, clip 0.05",
                   "tokens_per_step": tokens, "fresh_batch_every_step": True, "rotation_shards": c["shards"],
                   "hip_graph": bool(args.graph),
                   "optimizer": args.optimizer, "rotation": args.rotation,
                   "sgd_overlapped_with_backward": bool(args.sgd_overlap),
                   "sgd_fused_into_weight_gradient_products": bool(args.sgd_fused),
                   "logits_and_loss_fused": bool(args.fused_head_loss),
                   "wgrad_on_second_stream": bool(args.wgrad_overlap),
                   "next_layer_shards_read_ahead_into_cache": bool(ring.warm_ahead())},
        "roofline": dict(roof,
                     traffic=prof_ref["traffic_bytes"],
                     **{
                     "traffic_unit": "bytes per launch, read from the committed counter summary (not measured in this run)",
                     "from_profiles": prof_ref,
                     "algorithmic_bytes_per_launch": alg_bytes,
                     "algorithmic_bytes_formula": "per launch: (A rows x K + B rows x K) x 2 B, an operand that all shards "
                                                  "of the launch share counted once, + M x N x (output + addend + fused "
                                                  "update: 4 B master read, 4 B written, 2 B weight copy) ; averaged over "
                                                  "the launches of this variant in a step",
                     "kernel": dom_name,
                     "avg_launch_us": avg_ms * 1e3,
                     "launches_per_step": dom["launches"] // (5 if graph_stats is not None else prof_steps),
                     "flops_per_launch": dom["flops"] / dom["launches"],
                     "timed_in": ("HIP-graph replay of the step, both streams live: device time stamps per launch, times the "
                                  "ratio of rocprofv3's dispatch duration to that span in the committed profile"
                                  if graph_stats is not None else "eager launches, HIP events"),
                     "dispatch_over_execution_span": ratio,
                     "execution_span": span,
                     "eager_ms_per_step_with_event_pairs": eager_ms}),
        "gemm_kernels_in_graph_replay": graph_gemms,
        "measured_attainable": dict(peaks, dominant_kernel_frac_of_measured_gemm=achieved / peaks["gemm_bf16_4096_cubed_tflops"]),
        "step_mfma_frac": flops / dt / (PEAK["bf16_mfma_tflops"] * 1e12),
        "step_algorithmic_tflop": flops / 1e12,
        "all_gemm_kernels": {"ms_per_step": all_gemm_ms, "tflops": all_gemm_tflops},
        "shard_copy": None if copy is None else {"ms_per_step": copy["total_ms"] / prof_steps,
                                                 "gbs": copy["bytes"] / copy["total_ms"] / 1e6,
                                                 "frac_of_hbm_peak": copy["bytes"] / copy["total_ms"] / 1e6 / PEAK["hbm_gbs"]},
        "kernels": kernels,
        "peak_weight_bytes": {"rotated_weights_1x": rotated_weight_bytes(lm), "staging_two_slots": staging_bytes(dev),
                              "fp32_master_separate": opt.master_bytes(),
                              "ratio_weights_plus_staging_to_model": (rotated_weight_bytes(lm) + staging_bytes(dev)) /
                              rotated_weight_bytes(lm)},
        "loss_first_last": [first_loss, last_loss],
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(c)
    if whole and args.rotation == "direct":
        # The same step under the staged rotation: every window of shards copied home -> HBM slot by the copy kernel on
        # a side stream while the previous window's products read the other slot (the double buffer a multi-GPU ring
        # would fill from its neighbour).  Same model, same optimiser state layout, same timing recipe.
        ring.set_rotation_mode("staged")
        ring.set_warm_ahead(False)
        dt_s, g_s, _ = timed(2, args.steps)
        _lib.profile_enable(True)
        step()
        torch.cuda.synchronize()
        copy_s = _lib.profile_collect().get("shard_copy")
        _lib.profile_enable(False)
        staged = staging_bytes(dev)
        out["staged_rotation"] = {
            "ms_per_step": dt_s * 1e3, "tokens_per_s": tokens / dt_s, "staging_bytes": staged,
            "ratio_weights_plus_staging_to_model": (rotated_weight_bytes(lm) + staged) / rotated_weight_bytes(lm),
            "shard_copy_launches_per_step": None if copy_s is None else copy_s["launches"],
            "shard_copy_gbs": None if copy_s is None else copy_s["bytes"] / copy_s["total_ms"] / 1e6,
            "shard_copy_gbs_what": "bytes read + written by the copy kernel / its HIP-event time, one eager step",
            "hip_graph": bool(args.graph)}
        del g_s
        ring.set_rotation_mode("direct")
        ring.set_warm_ahead(args.warm_ahead)
    if whole and args.optimizer == "sgd":
        # The same step with the reference harness's own optimiser (benchmarks/rtp_benchmark.py:41-42, 185-186:
        # clip_grad_value_(0.05), then torch.optim.Adam(lr 1e-3)) instead of the SGD the headline asks for: gradients
        # are stored, fp32 moments live beside the fp32 master, one update launch over a device chunk table.
        for st in opt.stores:
            st.fused_sgd = None
        opt = RotatedAdam(lm, lr=1e-3, clip_value=0.05)
        dt_a, g_a, _ = timed(2, args.steps)
        out["reference_harness_optimizer"] = {
            "optimizer": "adam", "ms_per_step": dt_a * 1e3, "tokens_per_s": tokens / dt_a,
            "what": "clip 0.05 + Adam lr 1e-3 (torch.optim.Adam's arithmetic, fp32 moments), same model, rotation, "
                    "graph replay and fresh batch per step as the headline line",
            "hip_graph": bool(args.graph)}
        del g_a
    if whole:
        # The reference's other four configurations, one rotated layer each, fwd+bwd, same timing recipe.
        del g, lm, opt
        torch.cuda.empty_cache()
        others = {}
        for name in ("linear", "embedding", "attention", "moe"):
            r = layer_workload(name, args.steps, args.warmup, args.graph, not args.no_cpu_baseline, ring_result)
            others[name] = {"workload": r["config"]["workload"], "ms": r["value"], "dtype": r["dtype"],
                            "roofline": r["roofline"], "whole_layer": r["whole_layer"],
                            "cpu_baseline": r.get("cpu_baseline")}
        out["other_configs"] = others
    print(json.dumps(out))


if __name__ == "__main__":
    main()
