#!/usr/bin/env python3
"""Benchmark of the GGUF quantized-matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (BASELINE.json configs[1], the configuration the metric is quoted on): Q4_K decode matvec,
weight [14336 x 4096] (1x4096 -> 14336), batch 1, f32 activations ~N(0,1), weights ~N(0,0.02)
quantized to Q4_K on the device.  One "step" is one pass of the hot path over one activation batch,
i.e. one QMatMul::forward: the activation quantization (Q8_K, bit-identical to candle's CPU path) and
the matvec, which this library runs as ONE kernel.  Inputs are resident in HBM when the timed region
starts.  Steps rotate through a pool of distinct weight tensors larger than the 256 MB Infinity
Cache, so every step streams its 33 MB of weights from HBM.

At least 200 launches are timed after at least 20 warm-up launches, whatever --steps / --warmup say.

The JSON line carries, besides the driver contract fields:
  roofline      achieved algorithmic GB/s of the dominant (only) kernel of the step, from HIP events
                around back-to-back launches on the launch stream, against the 8 TB/s HBM peak, with
                the median / p10 / p90 over per-replay event pairs (one replay = one rotation of the pool);
                `traffic` = HBM bytes per launch from rocprofv3 FETCH_SIZE + WRITE_SIZE runs
                (read from the committed summary under profiles/, with the commit it was measured at)
  cpu_baseline  the C restatement of candle's CPU path (AVX2 dot products + column-split threads,
                oracle/cq_oracle_fast.c) timed on this box's host cores on bounded samples, for the headline
                configuration and for four more (Q8_0 4096x4096 batch 1, the headline shape at batch 16,
                Q6_K 4096x14336 at 128 rows, the matvecs of an 8B-shape decode step), with the CPU model and the thread count
  cfg1, cfg2_sweep, prefill, moe, decode_8b
                compact records of the other configurations: the Q8_0 4096 x 4096 matvec, the Q4_K batch sweep
                on both FFN shapes, the prefill matmuls at 128 / 512 / 2048 rows, the 48-layer MoE stack at
                1 / 16 / 256 tokens and the 8B-shape decoder

    python bench.py --pmc-mode     a handful of un-graphed launches of the step kernel plus one plain
                                   256 MiB device copy, for `rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE`
    python bench.py --workload prefill --pmc-mode --wdtype q4k --n 14336 --k 4096 --batch 2048
                                   the same for the prefill matmul: a few plain launches of QMatMul::forward
    python bench.py --workload prefill --wdtype q6k --n 4096 --k 14336 --batch 512
                                   the prefill matmul (other BASELINE configurations; not the headline line):
                                   TFLOP/s of QMatMul::forward and of its MFMA kernel against the 2.5 PFLOP/s
                                   dense f16 peak
    python bench.py --workload moe    the Qwen3-30B-A3B-shaped expert matmuls of one MoE layer at 1 / 16 / 256 tokens
    python bench.py --workload decode8b [--steps 256] [--prompt 512]
                                   the 8B-shape Q4_K_M decoder: prompt and decode tok/s against the weight-streaming
                                   roofline (8 TB/s / weight bytes per token)
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
MFMA_I8_PEAK_TOPS = 5000.0
MIN_TIMED_LAUNCHES = 200
MIN_WARMUP_LAUNCHES = 20
Q4K = 12
WDTYPES = {"q4_0": (2, 18, 32), "q8_0": (8, 34, 32), "q4k": (12, 144, 256), "q5k": (13, 176, 256), "q6k": (14, 210, 256),
           "q4_1": (3, 20, 32), "q5_0": (6, 22, 32), "q5_1": (7, 24, 32), "q2k": (10, 84, 256), "q3k": (11, 110, 256)}
FMT_NAMES = {"q4_0": "Q4_0", "q8_0": "Q8_0", "q4k": "Q4_K", "q5k": "Q5_K", "q6k": "Q6_K", "q4_1": "Q4_1", "q5_0": "Q5_0", "q5_1": "Q5_1",
             "q2k": "Q2_K", "q3k": "Q3_K"}
# formats whose prefill kernel runs on the int8 matrix cores (the others use the f16 ones)
I8_PREFILL = ("q4k", "q4_0", "q8_0", "q4_1", "q5_0", "q5_1")
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "q4k_decode_matvec_1x4096x14336_pmc.txt")


def algorithmic_bytes(n, k, m, type_size, block):
    """weights once + f32 activations in + f32 outputs (scratch traffic is not counted)."""
    return n * (k // block) * type_size + m * k * 4 + m * n * 4


def committed_traffic():
    """(HBM bytes per launch, commit) measured with rocprofv3 --pmc; the summary file holds the commands."""
    try:
        text = open(TRAFFIC_SUMMARY).read()
    except OSError:
        return None, None
    m = re.search(r"traffic_bytes_per_launch\s*=\s*(\d+)", text)
    c = re.search(r"measured_at_commit\s*=\s*([0-9a-f]+)", text)
    return (int(m.group(1)) if m else None), (c.group(1) if c else None)


def percentiles(samples):
    xs = sorted(samples)
    pick = lambda q: xs[min(len(xs) - 1, int(round(q * (len(xs) - 1))))]
    return {"median": pick(0.5), "p10": pick(0.1), "p90": pick(0.9), "n": len(xs)}


def quantized_weight(L, torch, dt, n, k, gen, dev, scale=0.02):
    """[n, k] f32 ~N(0, scale) quantized on the device, in row chunks so that the f32 source stays below 1 GB."""
    from candle_amd import _lib
    wbytes = L.cq_storage_bytes(dt, n * k)
    wq = torch.empty(wbytes, dtype=torch.uint8, device=dev)
    rows = max(1, min(n, (1 << 28) // k))
    row_bytes = wbytes // n
    for r0 in range(0, n, rows):
        r = min(rows, n - r0)
        wf = torch.randn((r, k), generator=gen, device=dev, dtype=torch.float32) * scale
        _lib.check("cq_quantize", L.cq_quantize(dt, wf.data_ptr(), wq.data_ptr() + r0 * row_bytes, r * k, None))
        torch.cuda.synchronize()
        del wf
    return wq


class Rotation:
    """One activation batch against a pool of distinct [n, k] weights, larger than the 256 MB Infinity Cache, captured as one
    HIP graph per rotation of the pool; timing with HIP events on the launch stream."""

    def __init__(self, L, torch, fmt, n, k, m, pool_mb, seed=1234):
        from candle_amd import _lib
        self.L, self.torch, self._lib = L, torch, _lib
        self.dt, self.ts, self.bs = WDTYPES[fmt]
        self.n, self.k, self.m = n, k, m
        dev = torch.device("cuda:0")
        self.wbytes = L.cq_storage_bytes(self.dt, n * k)
        self.alg_bytes = algorithmic_bytes(n, k, m, self.ts, self.bs)
        self.pool = max(2, (pool_mb * 1000 * 1000 + self.wbytes - 1) // self.wbytes)
        gen = torch.Generator(device=dev)
        gen.manual_seed(seed)
        self.weights = [quantized_weight(L, torch, self.dt, n, k, gen, dev) for _ in range(self.pool)]
        self.x = torch.randn((m, k), generator=gen, device=dev, dtype=torch.float32)
        self.dst = torch.empty((m, n), dtype=torch.float32, device=dev)
        self.ws_bytes = L.cq_qmatmul_workspace_bytes(self.dt, m, k, n)
        self.ws = torch.empty(max(self.ws_bytes, 256), dtype=torch.uint8, device=dev)
        self.stream = torch.cuda.Stream(device=dev)
        torch.cuda.synchronize()

    def step(self, i, sp):
        """QMatMul::forward: for up to 8 rows, activation quantization + matvec in one kernel."""
        self._lib.check("cq_qmatmul_forward", self.L.cq_qmatmul_forward(self.dt, self.weights[i % self.pool].data_ptr(), self.x.data_ptr(), 0,
                                                                       self.dst.data_ptr(), 0, self.m, self.k, self.n, self.ws.data_ptr(), self.ws_bytes, sp))

    def capture(self, fn, same_weight=False):
        torch = self.torch
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(self.stream):
            fn(0, self.stream.cuda_stream)          # warm the code path before capture
            self.stream.synchronize()
            with torch.cuda.graph(g, stream=self.stream):
                sp = torch.cuda.current_stream().cuda_stream
                for i in range(self.pool):
                    fn(0 if same_weight else i, sp)
        return g

    def run(self, graph, launches):
        reps = max(1, (launches + self.pool - 1) // self.pool)
        with self.torch.cuda.stream(self.stream):
            for _ in range(reps):
                graph.replay()
        return reps * self.pool

    def event_us(self, graph, launches, warmup):
        """Mean microseconds per launch over back-to-back replays (one event pair around all of them)."""
        torch = self.torch
        self.run(graph, warmup)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        with torch.cuda.stream(self.stream):
            e0.record(self.stream)
            done = self.run(graph, launches)
            e1.record(self.stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / done

    def replay_stats(self, graph, launches, warmup):
        """Microseconds per launch of every replay on its own (an event between replays): median / p10 / p90."""
        torch = self.torch
        self.run(graph, warmup)
        torch.cuda.synchronize()
        reps = max(8, (launches + self.pool - 1) // self.pool)
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(reps + 1)]
        with torch.cuda.stream(self.stream):
            ev[0].record(self.stream)
            for r in range(reps):
                graph.replay()
                ev[r + 1].record(self.stream)
        torch.cuda.synchronize()
        st = percentiles([ev[r].elapsed_time(ev[r + 1]) * 1e3 / self.pool for r in range(reps)])
        return {"median_us": round(st["median"], 3), "p10_us": round(st["p10"], 3), "p90_us": round(st["p90"], 3), "replays": st["n"],
                "launches_per_replay": self.pool}


def prefill_record(L, torch, fmt, n, k, m, steps=20, warmup=5, pmc=False):
    """QMatMul::forward with more than 8 activation rows: Q8_K / Q8_0 activation quantization kernel + MFMA matmul kernel."""
    from candle_amd import _lib
    dev = torch.device("cuda:0")
    dt, ts, bs = WDTYPES[fmt]
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)
    wq = quantized_weight(L, torch, dt, n, k, gen, dev)
    x = torch.randn((m, k), generator=gen, device=dev, dtype=torch.float32)
    dst = torch.empty((m, n), dtype=torch.float32, device=dev)
    ws_bytes = L.cq_qmatmul_workspace_bytes(dt, m, k, n)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    stream = torch.cuda.Stream(device=dev)
    sp = stream.cuda_stream

    def forward():
        _lib.check("cq_qmatmul_forward", L.cq_qmatmul_forward(dt, wq.data_ptr(), x.data_ptr(), 0, dst.data_ptr(), 0, m, k, n,
                                                              ws.data_ptr(), ws_bytes, sp))

    def quantize_only():
        _lib.check("cq_quantize_act", L.cq_quantize_act(dt, x.data_ptr(), 0, ws.data_ptr(), k, m, sp))

    # small grids split K into partial planes that a second kernel adds up (the workspace then holds those planes too)
    act_bytes = L.cq_act_scratch_bytes(dt, k, m)
    split_k = ws_bytes > act_bytes + ((m * n * 4 + 255) // 256) * 256

    if pmc:
        with torch.cuda.stream(stream):
            for _ in range(4):
                forward()
        torch.cuda.synchronize()
        return {"pmc_mode": True, "workload": "%s prefill [%d x %d] x [%d x %d]^T" % (fmt, m, k, n, k), "launches": 4}

    def event_us(fn, count):
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(count + 1)]
        with torch.cuda.stream(stream):
            for _ in range(warmup):
                fn()
            ev[0].record(stream)
            for i in range(count):
                fn()
                ev[i + 1].record(stream)
        torch.cuda.synchronize()
        return ev[0].elapsed_time(ev[count]) * 1e3 / count, percentiles([ev[i].elapsed_time(ev[i + 1]) * 1e3 for i in range(count)])

    with torch.cuda.stream(stream):
        for _ in range(warmup):
            forward()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    with torch.cuda.stream(stream):
        for _ in range(steps):
            forward()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    flops = 2.0 * m * n * k
    # the matrix-core part of what the forward launches (the split-K kernel and its reduction where K is split): the
    # forward's launches timed on the stream minus the activation quantization timed alone
    fwd_us, fst = event_us(forward, steps)
    q_us, _ = event_us(quantize_only, steps)
    kern_us = fwd_us - q_us
    kst = {key: fst[key] - q_us for key in ("median", "p10", "p90")}
    # the roofline is priced in algorithmic flop against the dense peak of the matrix-core type the kernel uses
    i8 = fmt in I8_PREFILL
    peak = MFMA_I8_PEAK_TOPS if i8 else MFMA_F16_PEAK_TFLOPS
    achieved = flops / (kern_us * 1e-6) / 1e12
    return {"fmt": fmt, "n": n, "k": k, "m": m, "steps": steps, "warmup": warmup, "forward_ms": round(ms, 5),
            "forward_TFLOPs": round(flops / (ms * 1e-3) / 1e12, 1), "kernel": "qmm_q4k_i8_kernel" if fmt == "q4k" else ("qmm_q0_i8_kernel<%s>" if i8 else "qmm_kernel<%s>") % fmt,
            "split_k": bool(split_k), "quantize_us": round(q_us, 2),
            "kernel_us": round(kern_us, 2), "kernel_median_us": round(kst["median"], 2), "kernel_p10_us": round(kst["p10"], 2),
            "kernel_p90_us": round(kst["p90"], 2), "kernel_TFLOPs": round(achieved, 1), "mfma": "i8" if i8 else "f16", "peak": peak,
            "frac": round(achieved / peak, 4)}


def prefill(args):
    import torch

    from candle_amd import _lib
    r = prefill_record(_lib.lib(), torch, args.wdtype, args.n, args.k, args.batch, max(args.steps, 20), max(args.warmup, 5), pmc=args.pmc_mode)
    if args.pmc_mode:
        print(json.dumps(r))
        return
    print(json.dumps({
        "metric": "%s prefill matmul TFLOP/s @%dx%d, M=%d" % (args.wdtype, args.n, args.k, args.batch), "value": r["forward_TFLOPs"],
        "unit": "TFLOP/s", "n_gpus": 1, "steps": r["steps"], "warmup": r["warmup"], "ms_per_step": r["forward_ms"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "i8 operands, i32 accumulate" if r["mfma"] == "i8" else "f16 operands, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": "%s prefill matmul [%d x %d] x [%d x %d]^T" % (args.wdtype, args.batch, args.k, args.n, args.k),
                   "step": "QMatMul::forward = activation quantization kernel + MFMA matmul kernel", "n": args.n, "k": args.k, "batch": args.batch},
        "roofline": {"bound": "mfma", "kernel": r["kernel"], "achieved": r["kernel_TFLOPs"], "peak": r["peak"], "unit": "TFLOP/s", "frac": r["frac"],
                     "traffic": None, "avg_kernel_us": r["kernel_us"], "median_us": r["kernel_median_us"], "p10_us": r["kernel_p10_us"],
                     "p90_us": r["kernel_p90_us"]},
    }))


def decode8b(args):
    """BASELINE configs[3]: random-init Llama-3-8B-shaped decoder, Q4_K_M mix, 512-token prefill then greedy decode, batch 1."""
    import torch

    from candle_amd.quantized_llama import Config, ModelWeights

    cfg = Config.llama3_8b()
    cfg.n_layer = args.layers
    t0 = time.perf_counter()
    model = ModelWeights.random_init(cfg, seed=1234)
    torch.cuda.synchronize()
    t_init = time.perf_counter() - t0
    gen = torch.Generator()
    gen.manual_seed(99)
    prompt = torch.randint(0, cfg.vocab, (args.prompt,), generator=gen).tolist()
    n_new = args.steps if args.steps else 256
    model.generate_greedy(prompt, min(n_new, 8))                      # warm-up: code paths, graph capture
    res = model.generate_greedy(prompt, n_new)
    # the same run from a step captured once for the whole context (more, shorter attention splits per head)
    model.generate_greedy(prompt, min(n_new, 8), max_kv=cfg.ctx)
    res_ctx = model.generate_greedy(prompt, n_new, max_kv=cfg.ctx)
    # (another split count sums the attention in another order: on random weights the greedy tokens may part ways at a near tie)
    same = next((i for i, (a, b) in enumerate(zip(res["tokens"], res_ctx["tokens"])) if a != b), len(res["tokens"]))
    wbytes = model.weight_bytes_per_token()
    steps = res["decode_steps"]
    tok_s = steps / res["decode_seconds"]
    # KV bytes read per decode step, averaged over the positions of the run (f32 cache, K and V)
    mean_pos = args.prompt + (n_new + 1) / 2.0
    kv_bytes = 2 * cfg.n_layer * cfg.n_kv_head * cfg.head_dim * 4 * mean_pos
    roof_tok_s = HBM_PEAK_GBPS * 1e9 / wbytes
    out = {
        "metric": "8B-shape Q4_K_M decode tok/s (batch 1, greedy)", "value": round(tok_s, 1), "unit": "tok/s", "n_gpus": 1,
        "steps": steps, "warmup": 8, "ms_per_step": round(1e3 / tok_s, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "i8 dot products, f32 glue", "data": "synthetic",
        "config": {"workload": "Llama-3-8B shape, %d layers, hidden 4096, 32 q / 8 kv heads, head_dim 128, FFN 14336, vocab 128256; "
                               "attn_v / ffn_down Q6_K, rest and head Q4_K; f32 embedding table; rope theta 500000, rms eps 1e-5; "
                               "%d random prompt tokens prefilled in one forward, then %d greedy single-token steps replayed from one HIP graph"
                               % (cfg.n_layer, args.prompt, steps),
                   "ctx": cfg.ctx, "prompt_tokens": args.prompt},
        "prompt_tok_s": round(args.prompt / res["prompt_seconds"], 1),
        "captured_for_kv": args.prompt + n_new, "tok_s_captured_for_ctx": round(res_ctx["decode_steps"] / res_ctx["decode_seconds"], 1),
        "captured_for_ctx_equal_leading_tokens": same,
        "weight_bytes_per_token": wbytes, "kv_bytes_per_token_mean": int(kv_bytes),
        "roofline": {"bound": "hbm", "kernel": "whole decode step (weights streamed once per token)",
                     "achieved": round((wbytes + kv_bytes) * tok_s / 1e9, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round((wbytes + kv_bytes) * tok_s / 1e9 / HBM_PEAK_GBPS, 4), "traffic": None,
                     "roofline_tok_s_weights_only": round(roof_tok_s, 1), "frac_of_roofline_tok_s": round(tok_s / roof_tok_s, 4)},
        "init_seconds": round(t_init, 1),
    }
    del model
    torch.cuda.empty_cache()
    return out


def moe(args):
    """BASELINE configs[4]: Qwen3-30B-A3B-shaped MoE layer stack (48 layers, 128 experts, top-8, hidden 2048, expert FFN 768, Q4_K,
    16 GB of expert weights, every layer with weights of its own): the three expert matmuls of each layer (gate, up on
    [tokens, hidden]; down on [tokens*8, ffn]) through QTensor::indexed_moe_forward, and the whole layers through
    FusedMoeGGUF::forward, for 1 / 16 / 256 tokens, each as one HIP graph over all layers."""
    import torch

    from candle_amd import _lib
    from candle_amd.fused_moe import FusedMoeGGUF
    from candle_amd.quantized import GgmlDType, QStorage, QTensor

    L = _lib.lib()
    dev = torch.device("cuda:0")
    E, H, F, TOPK, NL = 128, 2048, 768, 8, args.moe_layers
    wdt, block_bytes, _ = WDTYPES[args.wdtype]              # (--wdtype: the experts' format, Q4_K unless given)
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)
    gate = [quantized_weight(L, torch, wdt, E * F, H, gen, dev) for _ in range(NL)]
    up = [quantized_weight(L, torch, wdt, E * F, H, gen, dev) for _ in range(NL)]
    down = [quantized_weight(L, torch, wdt, E * H, F, gen, dev) for _ in range(NL)]
    router = torch.randn((E, H), generator=gen, device=dev)

    def qt(buf, n, k):
        return QTensor.new(QStorage(buf, GgmlDType(wdt)), (E, n, k))

    fused = [FusedMoeGGUF(router, qt(gate[i], F, H), qt(up[i], F, H), qt(down[i], H, F), True, TOPK) for i in range(NL)]
    reps, warm = max(1, (MIN_TIMED_LAUNCHES + NL - 1) // NL), max(1, (MIN_WARMUP_LAUNCHES + NL - 1) // NL)
    results = []
    for tokens in [int(t) for t in args.moe_tokens.split(",")]:
        x = torch.randn((tokens, H), generator=gen, device=dev)
        _, ids = torch.topk(torch.softmax(x @ router.t(), -1), TOPK, dim=-1)
        ids32 = ids.to(torch.int32).contiguous()
        distinct = int(torch.unique(ids).numel())
        xg = x.reshape(tokens, 1, H).contiguous()
        h = torch.randn((tokens, TOPK, F), generator=gen, device=dev)
        o1, o2 = torch.empty((tokens, TOPK, F), device=dev), torch.empty((tokens, TOPK, F), device=dev)
        o3 = torch.empty((tokens, TOPK, H), device=dev)
        nws = max(L.cq_indexed_moe_workspace_bytes(wdt, E, F, H, tokens, TOPK, 1), L.cq_indexed_moe_workspace_bytes(wdt, E, H, F, tokens, TOPK, TOPK))
        ws = torch.empty(nws, dtype=torch.uint8, device=dev)

        def layer(i, sp):
            for w, src, dst, n, k, d1 in ((gate[i], xg, o1, F, H, 1), (up[i], xg, o2, F, H, 1), (down[i], h, o3, H, F, TOPK)):
                _lib.check("cq_indexed_moe_forward", L.cq_indexed_moe_forward(wdt, w.data_ptr(), src.data_ptr(), ids32.data_ptr(), dst.data_ptr(),
                                                                              E, n, k, tokens, TOPK, d1, ws.data_ptr(), nws, sp))

        st = torch.cuda.Stream(device=dev)
        x3 = x.reshape(1, tokens, H)
        y = torch.empty((tokens, H), device=dev)

        def timed(run_layer):
            """per-layer microseconds of a graph over all NL layers: mean, and median / p10 / p90 over the replays"""
            with torch.cuda.stream(st):
                run_layer(0)
                st.synchronize()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=st):
                    for i in range(NL):
                        run_layer(i)
                for _ in range(warm):
                    g.replay()
                st.synchronize()
                ev = [torch.cuda.Event(enable_timing=True) for _ in range(reps + 1)]
                ev[0].record(st)
                for r in range(reps):
                    g.replay()
                    ev[r + 1].record(st)
                st.synchronize()
            pst = percentiles([ev[r].elapsed_time(ev[r + 1]) * 1e3 / NL for r in range(reps)])
            return ev[0].elapsed_time(ev[reps]) * 1e3 / (reps * NL), pst

        us, ust = timed(lambda i: layer(i, torch.cuda.current_stream().cuda_stream))
        # the whole layer as FusedMoeGGUF::forward runs it: router + softmax + top-k, sort by expert, three grouped
        # matmuls (moe_gemm_gguf), silu(gate) * up, sum over top-k
        fused_us, fst = timed(lambda i: fused[i].forward(x3, tokens > 1, out=y))
        alg = distinct * 3 * (F * H // 256) * block_bytes
        results.append({"tokens": tokens, "distinct_experts": distinct, "layer_us": round(us, 1), "layer_median_us": round(ust["median"], 1),
                        "layer_p10_us": round(ust["p10"], 1), "layer_p90_us": round(ust["p90"], 1), "algorithmic_MB": round(alg / 1e6, 1),
                        "GBps": round(alg / us / 1e3, 1), "frac_of_hbm_peak": round(alg / us / 1e3 / HBM_PEAK_GBPS, 4),
                        "fused_moe_layer_us": round(fused_us, 1), "fused_moe_layer_median_us": round(fst["median"], 1),
                        "tok_s_%d_layers_fused" % NL: round(tokens / (NL * fused_us * 1e-6), 1), "timed_layer_launches": reps * NL})
    out = {"metric": "Qwen3-30B-A3B-shape MoE layer, expert matmuls (%s, 128 experts, top-8)" % FMT_NAMES[args.wdtype], "unit": "us per layer", "n_gpus": 1,
           "data": "synthetic", "config": {"workload": "gate + up [tokens, 2048] -> 768 and down [tokens*8, 768] -> 2048 via indexed_moe_forward, "
                                                       "%d layers with distinct weights (%.1f GB) in one HIP graph; fused_moe_layer_us: the same "
                                                       "layers through FusedMoeGGUF::forward (router, top-k, sort, moe_gemm_gguf x3, "
                                                       "silu*up, sum over top-k)" % (NL, NL * 3 * E * (F * H // 256) * block_bytes / 1e9), "layers": NL},
           "results": results}
    del gate, up, down, fused
    torch.cuda.empty_cache()
    return out


def cpu_info():
    """(model name, physical cores this process may run on, threads used): threads = physical cores, at most the 16 the box allots."""
    model, phys = "unknown", set()
    try:
        allowed = os.sched_getaffinity(0)
        cur = {}
        for line in open("/proc/cpuinfo"):
            if ":" in line:
                key, val = [t.strip() for t in line.split(":", 1)]
                cur[key] = val
            elif cur:
                if int(cur.get("processor", -1)) in allowed:
                    phys.add((cur.get("physical id", "0"), cur.get("core id", cur.get("processor"))))
                model = cur.get("model name", model)
                cur = {}
        if cur and int(cur.get("processor", -1)) in allowed:
            phys.add((cur.get("physical id", "0"), cur.get("core id", cur.get("processor"))))
    except (OSError, ValueError):
        pass
    n_phys = max(1, len(phys))
    return model, n_phys, max(1, min(n_phys, 16))


def cpu_matmul_baseline(torch, fmt, n, k, m, threads, seconds, copies, seed=77):
    """The C restatement of candle's CPU QMatMul::forward (Q8_K / Q8_0 activation quantization + AVX2 vec_dot + column split over
    threads) on host copies of GPU-quantized weights, rotated so that the weights come from DRAM; time-bounded."""
    import oracle
    from candle_amd import _lib
    L = _lib.lib()
    dev = torch.device("cuda:0")
    dt, ts, bs = WDTYPES[fmt]
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    hw = [quantized_weight(L, torch, dt, n, k, gen, dev).cpu().numpy() for _ in range(copies)]
    hx = torch.randn((m, k), generator=gen, device=dev).cpu().numpy()
    oracle.matmul_fast(dt, hx, hw[0], n, threads)
    t0 = time.perf_counter()
    it = 0
    while time.perf_counter() - t0 < seconds or it < 2:
        oracle.matmul_fast(dt, hx, hw[it % copies], n, threads)
        it += 1
    dt_s = (time.perf_counter() - t0) / it
    alg = algorithmic_bytes(n, k, m, ts, bs)
    return {"workload": "%s [%d x %d] x %d rows" % (FMT_NAMES[fmt], n, k, m), "ms_per_call": round(dt_s * 1e3, 4), "GBps": round(alg / dt_s / 1e9, 2),
            "GFLOPs": round(2.0 * m * n * k / dt_s / 1e9, 1), "calls": it, "seconds": round(dt_s * it, 1), "weight_copies": copies}


def cpu_decode_baseline(torch, threads, seconds_each=1.0):
    """cfg4 on the CPU restatement: the eight matvecs of one decode step of the 8B-shape Q4_K_M model (seven per layer and the
    output head), each timed on its own at one activation row; a token is 32 layers plus the head (the f32 glue — norms,
    rope, attention, silu — is left out, so this flatters the CPU)."""
    shapes = [("attention_wq", "q4k", 4096, 4096), ("attention_wk", "q4k", 1024, 4096), ("attention_wv", "q6k", 1024, 4096),
              ("attention_wo", "q4k", 4096, 4096), ("feed_forward_w1", "q4k", 14336, 4096), ("feed_forward_w3", "q4k", 14336, 4096),
              ("feed_forward_w2", "q6k", 4096, 14336), ("output", "q4k", 128256, 4096)]
    per = {}
    for name, fmt, n, k in shapes:
        r = cpu_matmul_baseline(torch, fmt, n, k, 1, threads, seconds_each, copies=2 if n > 100000 else 6)
        per[name] = r["ms_per_call"]
    layer_ms = sum(v for kname, v in per.items() if kname != "output")
    token_ms = 32 * layer_ms + per["output"]
    return {"workload": "8B-shape Q4_K_M decode, matvecs only: 32 x (wq, wk, wv, wo, w1, w3, w2) + output head, one row",
            "ms_per_matvec": per, "layer_ms": round(layer_ms, 3), "token_ms": round(token_ms, 2), "tok_s": round(1e3 / token_ms, 1)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--workload", choices=["decode", "prefill", "decode8b", "moe"], default="decode")
    ap.add_argument("--layers", type=int, default=32, help="--workload decode8b: number of decoder layers")
    ap.add_argument("--prompt", type=int, default=512, help="--workload decode8b: prompt tokens")
    ap.add_argument("--moe-tokens", default="1,16,256", help="--workload moe: token counts, comma separated")
    ap.add_argument("--moe-layers", type=int, default=48, help="--workload moe: layers, each with its own expert weights (340 MB per layer)")
    ap.add_argument("--wdtype", choices=sorted(WDTYPES), default="q4k",
                    help="weight format of --workload prefill / decode (the metric is quoted on q4k; other formats skip the other configurations)")
    ap.add_argument("--n", type=int, default=14336)
    ap.add_argument("--k", type=int, default=4096)
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--pool-mb", type=int, default=1280, help="distinct weight bytes rotated through (MB)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=8.0, help="CPU time of the headline baseline; the three others take 3 s each")
    ap.add_argument("--pmc-mode", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="only the headline step: skip the context numbers and the other configurations")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (every configuration of the metric is single-GPU); use --gpus 1")
    if args.workload == "decode8b":
        print(json.dumps(decode8b(args)))
        return
    if args.workload == "moe":
        print(json.dumps(moe(args)))
        return
    if args.steps is None:
        args.steps = 4000 if args.workload == "decode" else 50
    if args.warmup is None:
        args.warmup = 400 if args.workload == "decode" else 5
    if args.workload == "prefill":
        return prefill(args)
    # the protocol's floor, whatever the flags say
    args.steps = max(args.steps, MIN_TIMED_LAUNCHES)
    args.warmup = max(args.warmup, MIN_WARMUP_LAUNCHES)

    import torch

    from candle_amd import _lib

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    L = _lib.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    n, k, m = args.n, args.k, args.batch
    fmt = FMT_NAMES[args.wdtype]
    headline = args.wdtype == "q4k" and (n, k, m) == (14336, 4096, 1)
    if not headline:
        args.no_cpu_baseline = True

    # ---- synthetic inputs, resident in HBM --------------------------------------------------
    rot = Rotation(L, torch, args.wdtype, n, k, m, 270 if args.pmc_mode else args.pool_mb)
    pool, alg_bytes, wbytes, stream = rot.pool, rot.alg_bytes, rot.wbytes, rot.stream

    if args.pmc_mode:
        # plain launches (one dispatch row per kernel in the counter CSV) + a copy of known size
        with torch.cuda.stream(stream):
            for i in range(2 * pool):
                rot.step(i, stream.cuda_stream)
            a = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
            b = torch.empty_like(a)
            stream.synchronize()
            for _ in range(4):
                b.copy_(a)
        torch.cuda.synchronize()
        print(json.dumps({"pmc_mode": True, "copy_bytes": 256 << 20, "step_algorithmic_bytes": alg_bytes, "step_launches": 2 * pool}))
        return

    # The step is a few microseconds of GPU work: one rotation over the pool is captured in a HIP graph
    # so that host launch latency is not what gets measured.
    g_step = rot.capture(rot.step)

    # ---- timed region: K steps (rounded up to whole rotations of the pool), wall clock ------------
    rot.run(g_step, args.warmup)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    done = rot.run(g_step, args.steps)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / done
    value = alg_bytes / (ms_per_step * 1e-3) / 1e9

    # ---- dominant kernel (the step IS one kernel): HIP events around the same back-to-back launches ----
    kern_us = rot.event_us(g_step, args.steps, args.warmup)
    stats = rot.replay_stats(g_step, args.steps, args.warmup)
    achieved = alg_bytes / (kern_us * 1e-6) / 1e9
    # context numbers, labelled: the same kernel with the weights resident in the Infinity Cache (one
    # tensor reused), and the matvec over activations quantized beforehand by cq_quantize_act
    extra = None
    if not args.no_extra:
        def matvec_prequantized(i, sp):
            _lib.check("cq_matvec", L.cq_matvec(rot.dt, rot.weights[i % pool].data_ptr(), rot.ws.data_ptr(), rot.dst.data_ptr(), 0, k, n, m, n, sp))

        resident_us = rot.event_us(rot.capture(rot.step, same_weight=True), args.steps, args.warmup)
        _lib.check("cq_quantize_act", L.cq_quantize_act(rot.dt, rot.x.data_ptr(), 0, rot.ws.data_ptr(), k, m, None))
        torch.cuda.synchronize()
        preq_us = rot.event_us(rot.capture(matvec_prequantized), args.steps, args.warmup)
        extra = {"infinity_cache_resident_us": round(resident_us, 3),
                 "infinity_cache_resident_GBps": round(alg_bytes / (resident_us * 1e-6) / 1e9, 1),
                 "prequantized_matvec_us": round(preq_us, 3),
                 "prequantized_matvec_GBps": round(alg_bytes / (preq_us * 1e-6) / 1e9, 1)}
        # the yardstick: a kernel that only reads the same rotated tensors, same launch shape
        bench_lib = _lib.bench_lib()
        if bench_lib is not None:
            sink = torch.zeros(4, dtype=torch.int32, device=dev)
            read_bytes = wbytes - wbytes % 16

            def plain_read(i, sp):
                _lib.check("cq_bench_read", bench_lib.cq_bench_read(rot.weights[i % pool].data_ptr(), read_bytes, sink.data_ptr(), sp))

            def plain_read_best(i, sp):
                _lib.check("cq_bench_read_best", bench_lib.cq_bench_read_best(rot.weights[i % pool].data_ptr(), read_bytes, sink.data_ptr(), sp))

            read_us = rot.event_us(rot.capture(plain_read), args.steps, args.warmup)
            best_us = rot.event_us(rot.capture(plain_read_best), args.steps, args.warmup)
            # plain_read: 256 x 1024 threads like the matvec, four loads in flight; plain_read_best: the fastest shape of a sweep
            extra.update({"plain_read_us": round(read_us, 3), "plain_read_GBps": round(read_bytes / (read_us * 1e-6) / 1e9, 1),
                          "plain_read_best_shape_us": round(best_us, 3),
                          "plain_read_best_shape_GBps": round(read_bytes / (best_us * 1e-6) / 1e9, 1)})

    traffic, traffic_commit = committed_traffic() if headline else (None, None)
    out = {
        "metric": "%s matvec GB/s @%dx%d (decode, batch %d)" % (fmt, k, n, m),
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": done,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "i8",
        "data": "synthetic",
        "config": {"workload": "%s decode matvec 1x%d->%d, weight [%d x %d] %s, batch %d, %d distinct weight tensors rotated (%.2f GB)"
                               % (fmt, k, n, n, k, fmt, m, pool, pool * wbytes / 1e9),
                   "step": "QMatMul::forward = %s activation quantization + matvec in one kernel, launches captured in a HIP graph"
                           % ("Q8_K" if rot.bs == 256 else "Q8_0"),
                   "n": n, "k": k, "batch": m},
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "roofline": {"bound": "hbm", "kernel": "%s<%s, %d row%s, fused f32 activations>" % (
                         ("qms_kernel_dw" if m == 1 else "qms_rows2_kernel") if args.wdtype in ("q4k", "q5k", "q6k", "q4_0", "q8_0") and m <= 2
                         else "qmv_kernel", fmt, m, "" if m == 1 else "s"),
                     "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": traffic, "traffic_commit": traffic_commit, "avg_kernel_us": round(kern_us, 3), "median_us": stats["median_us"],
                     "p10_us": stats["p10_us"], "p90_us": stats["p90_us"], "timed_launches": stats["replays"] * pool,
                     "replays": stats["replays"], "algorithmic_bytes_per_launch": alg_bytes},
        "extra": extra,
    }
    del rot, g_step
    torch.cuda.empty_cache()

    if not args.no_extra and headline:
        out.update(other_configurations(L, torch, args))

    if not args.no_cpu_baseline:
        model, n_phys, threads = cpu_info()
        head = cpu_matmul_baseline(torch, "q4k", n, k, 1, threads, args.cpu_seconds, copies=8)
        out["cpu_baseline"] = {"value": head["GBps"], "unit": "GB/s", "cores": threads, "kind": "port",
                               "sample": "%d calls of the same 1x%d->%d Q4_K matvec over %d rotated host weight copies (%.1f s); "
                                         "C restatement of candle's CPU path: Q8_K activation quantize + AVX2 vec_dot + column split over threads"
                                         % (head["calls"], k, n, head["weight_copies"], head["seconds"]),
                               "ms_per_call": head["ms_per_call"], "cpu_model": model, "physical_cores_available": n_phys,
                               "threads_rule": "physical cores, at most the 16 this box allots to one GPU",
                               "others": {"cfg1_q8_0_4096x4096_b1": cpu_matmul_baseline(torch, "q8_0", 4096, 4096, 1, threads, 3.0, copies=16),
                                          "cfg2_q4k_14336x4096_b16": cpu_matmul_baseline(torch, "q4k", 14336, 4096, 16, threads, 3.0, copies=8),
                                          "cfg3_q6k_4096x14336_m128": cpu_matmul_baseline(torch, "q6k", 4096, 14336, 128, threads, 3.0, copies=4),
                                          "cfg4_decode_8b": cpu_decode_baseline(torch, threads)}}
    print(json.dumps(out))


def other_configurations(L, torch, args):
    """Compact records of the configurations the metric is not quoted on."""
    out = {}
    # cfg1: the single Q8_0 matvec, 4096 x 4096, batch 1
    rot = Rotation(L, torch, "q8_0", 4096, 4096, 1, 600)
    g = rot.capture(rot.step)
    us = rot.event_us(g, 2000, 200)
    st = rot.replay_stats(g, 2000, 200)
    out["cfg1"] = {"workload": "Q8_0 matvec 1x4096->4096, %d weights rotated" % rot.pool, "us": round(us, 3), "median_us": st["median_us"],
                   "p10_us": st["p10_us"], "p90_us": st["p90_us"], "GBps": round(rot.alg_bytes / us / 1e3, 1),
                   "frac_of_hbm_peak": round(rot.alg_bytes / us / 1e3 / HBM_PEAK_GBPS, 4)}
    del rot, g
    torch.cuda.empty_cache()
    # cfg2: the Q4_K batch sweep on both FFN shapes (3 .. 16 rows: the batched matrix-core matvec; the first shape also at 32 and 64
    # rows, which run as sets of 16 rows through the same formulation)
    sweep = []
    for (n, k) in ((14336, 4096), (4096, 14336)):
        for b in (1, 2, 4, 8, 16) + ((32, 64) if k <= 4096 else ()):
            rot = Rotation(L, torch, "q4k", n, k, b, args.pool_mb)          # the headline's pool: 39 launches per graph replay
            g = rot.capture(rot.step)
            us = rot.event_us(g, 1000, 100)
            st = rot.replay_stats(g, 1000, 100)
            sweep.append({"n": n, "k": k, "batch": b, "us": round(us, 3), "median_us": st["median_us"], "p10_us": st["p10_us"], "p90_us": st["p90_us"],
                          "GBps": round(rot.alg_bytes / us / 1e3, 1), "frac_of_hbm_peak": round(rot.alg_bytes / us / 1e3 / HBM_PEAK_GBPS, 4)})
            del rot, g
            torch.cuda.empty_cache()
    out["cfg2_sweep"] = sweep
    # cfg3: prefill at 128 / 512 / 2048 rows
    pf = []
    for fmt, n, k in (("q6k", 4096, 14336), ("q5k", 14336, 4096), ("q4_0", 4096, 14336), ("q4_0", 14336, 4096), ("q4k", 14336, 4096)):
        for m in (128, 512, 2048):
            pf.append(prefill_record(L, torch, fmt, n, k, m, steps=20, warmup=5))
            torch.cuda.empty_cache()
    out["prefill"] = pf
    # cfg4: the 8B-shape decoder (same protocol as --workload decode8b)
    r = decode8b(argparse.Namespace(layers=32, prompt=512, steps=256))
    out["decode_8b"] = {"tok_s": r["value"], "ms_per_token": r["ms_per_step"], "prompt_tok_s": r["prompt_tok_s"],
                        "captured_for_kv": r["captured_for_kv"], "tok_s_captured_for_ctx": r["tok_s_captured_for_ctx"],
                        "frac_of_roofline_tok_s": r["roofline"]["frac_of_roofline_tok_s"],
                        "roofline_tok_s": r["roofline"]["roofline_tok_s_weights_only"],
                        "weight_bytes_per_token": r["weight_bytes_per_token"], "workload": r["config"]["workload"]}
    # cfg5: the 48-layer MoE stack
    mo = moe(argparse.Namespace(moe_layers=48, moe_tokens="1,16,256", wdtype="q4k"))
    out["moe"] = {"workload": mo["config"]["workload"], "results": mo["results"]}
    return out


if __name__ == "__main__":
    main()
