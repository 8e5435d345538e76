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

The JSON line carries, besides the driver contract fields:
  roofline      achieved algorithmic GB/s of the dominant (only) kernel of the step, from HIP events
                around back-to-back launches on the launch stream, against the 8 TB/s HBM peak;
                `traffic` = HBM bytes per launch from rocprofv3 FETCH_SIZE + WRITE_SIZE runs
                (read from the committed summary under profiles/ when present)
  cpu_baseline  the C restatement of candle's CPU path (AVX2 dot products + column-split threads,
                oracle/cq_oracle_fast.c) timed on this box's host cores on a bounded sample

    python bench.py --pmc-mode     a handful of un-graphed launches of the step kernel plus one plain
                                   256 MiB device copy, for `rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE`
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
Q4K = 12
WDTYPES = {"q4_0": (2, 18, 32), "q8_0": (8, 34, 32), "q4k": (12, 144, 256), "q5k": (13, 176, 256), "q6k": (14, 210, 256),
           "q4_1": (3, 20, 32), "q5_0": (6, 22, 32), "q5_1": (7, 24, 32), "q2k": (10, 84, 256), "q3k": (11, 110, 256)}
FMT_NAMES = {"q4_0": "Q4_0", "q8_0": "Q8_0", "q4k": "Q4_K", "q5k": "Q5_K", "q6k": "Q6_K", "q4_1": "Q4_1", "q5_0": "Q5_0", "q5_1": "Q5_1",
             "q2k": "Q2_K", "q3k": "Q3_K"}
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "q4k_decode_matvec_1x4096x14336_pmc.txt")


def algorithmic_bytes(n, k, m, type_size, block):
    """weights once + f32 activations in + f32 outputs (scratch traffic is not counted)."""
    return n * (k // block) * type_size + m * k * 4 + m * n * 4


def committed_traffic():
    """HBM bytes per launch measured with rocprofv3 --pmc (see the summary file for the commands)."""
    try:
        m = re.search(r"traffic_bytes_per_launch\s*=\s*(\d+)", open(TRAFFIC_SUMMARY).read())
        return int(m.group(1)) if m else None
    except OSError:
        return None


def prefill(args):
    """QMatMul::forward with more than 8 activation rows: Q8_K / Q8_0 activation quantization kernel + MFMA matmul kernel."""
    import torch

    from candle_amd import _lib

    L = _lib.lib()
    dev = torch.device("cuda:0")
    dt, ts, bs = WDTYPES[args.wdtype]
    n, k, m = args.n, args.k, args.batch
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)
    wbytes = L.cq_storage_bytes(dt, n * k)
    wf = torch.randn((n, k), generator=gen, device=dev, dtype=torch.float32) * 0.02
    wq = torch.empty(wbytes, dtype=torch.uint8, device=dev)
    _lib.check("cq_quantize", L.cq_quantize(dt, wf.data_ptr(), wq.data_ptr(), n * k, None))
    del wf
    x = torch.randn((m, k), generator=gen, device=dev, dtype=torch.float32)
    dst = torch.empty((m, n), dtype=torch.float32, device=dev)
    ws_bytes = L.cq_qmatmul_workspace_bytes(dt, m, k, n)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    stream = torch.cuda.Stream(device=dev)
    sp = stream.cuda_stream

    def forward():
        _lib.check("cq_qmatmul_forward", L.cq_qmatmul_forward(dt, wq.data_ptr(), x.data_ptr(), 0, dst.data_ptr(), 0, m, k, n,
                                                              ws.data_ptr(), ws_bytes, sp))

    def matmul_only():
        _lib.check("cq_matmul", L.cq_matmul(dt, wq.data_ptr(), ws.data_ptr(), dst.data_ptr(), k, n, m, n, sp))

    def event_us(fn, steps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        with torch.cuda.stream(stream):
            for _ in range(args.warmup):
                fn()
            e0.record(stream)
            for _ in range(steps):
                fn()
            e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / steps

    steps = args.steps
    with torch.cuda.stream(stream):
        for _ in range(args.warmup):
            forward()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    with torch.cuda.stream(stream):
        for _ in range(steps):
            forward()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    flops = 2.0 * m * n * k
    kern_us = event_us(matmul_only, steps)
    # Q4_K runs on the int8 matrix cores (two int8 MACs per algorithmic MAC: the scale is split in two), the other formats
    # on the f16 ones; the roofline is priced in algorithmic flop against the peak of the unit used
    i8 = args.wdtype == "q4k"
    peak = MFMA_I8_PEAK_TOPS if i8 else MFMA_F16_PEAK_TFLOPS
    achieved = flops / (kern_us * 1e-6) / 1e12
    print(json.dumps({
        "metric": "%s prefill matmul TFLOP/s @%dx%d, M=%d" % (args.wdtype, n, k, m), "value": round(flops / (ms * 1e-3) / 1e12, 1),
        "unit": "TFLOP/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup, "ms_per_step": round(ms, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "i8 operands, i32 accumulate" if i8 else "f16 operands, f32 accumulate", "data": "synthetic",
        "config": {"workload": "%s prefill matmul [%d x %d] x [%d x %d]^T" % (args.wdtype, m, k, n, k),
                   "step": "QMatMul::forward = activation quantization kernel + MFMA matmul kernel", "n": n, "k": k, "batch": m},
        "roofline": {"bound": "mfma", "kernel": "qmm_q4k_i8_kernel" if i8 else "qmm_kernel<%s>" % args.wdtype, "achieved": round(achieved, 1),
                     "peak": peak, "unit": "TFLOP/s", "frac": round(achieved / peak, 4), "traffic": None, "avg_kernel_us": round(kern_us, 2)},
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
    """BASELINE configs[4]: Qwen3-30B-A3B-shaped MoE layer (128 experts, top-8, hidden 2048, expert FFN 768, Q4_K):
    the three expert matmuls of one layer (gate, up on [tokens, hidden]; down on [tokens*8, ffn]) through
    QTensor::indexed_moe_forward, rotated over several distinct layers, for 1 / 16 / 256 tokens."""
    import torch

    from candle_amd import _lib

    L = _lib.lib()
    dev = torch.device("cuda:0")
    E, H, F, TOPK, NL = 128, 2048, 768, 8, 6
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)

    def experts(n, k):
        nb = L.cq_storage_bytes(Q4K, E * n * k)
        w = torch.empty(nb, dtype=torch.uint8, device=dev)
        for e in range(E):
            wf = torch.randn((n, k), generator=gen, device=dev) * 0.02
            _lib.check("cq_quantize", L.cq_quantize(Q4K, wf.data_ptr(), w.data_ptr() + e * (nb // E), n * k, None))
        torch.cuda.synchronize()
        return w

    gate, up, down = [experts(F, H) for _ in range(NL)], [experts(F, H) for _ in range(NL)], [experts(H, F) for _ in range(NL)]
    router = torch.randn((E, H), generator=gen, device=dev)
    from candle_amd.fused_moe import FusedMoeGGUF
    from candle_amd.quantized import GgmlDType, QStorage, QTensor

    def qt(buf, n, k):
        return QTensor.new(QStorage(buf, GgmlDType.Q4K), (E, n, k))

    fused = [FusedMoeGGUF(router, qt(gate[i], F, H), qt(up[i], F, H), qt(down[i], H, F), True, TOPK) for i in range(NL)]
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
        nws = max(L.cq_indexed_moe_workspace_bytes(Q4K, E, F, H, tokens, TOPK, 1), L.cq_indexed_moe_workspace_bytes(Q4K, E, H, F, tokens, TOPK, TOPK))
        ws = torch.empty(nws, dtype=torch.uint8, device=dev)

        def layer(i, sp):
            for w, src, dst, n, k, d1 in ((gate[i % NL], xg, o1, F, H, 1), (up[i % NL], xg, o2, F, H, 1), (down[i % NL], h, o3, H, F, TOPK)):
                _lib.check("cq_indexed_moe_forward", L.cq_indexed_moe_forward(Q4K, w.data_ptr(), src.data_ptr(), ids32.data_ptr(), dst.data_ptr(),
                                                                              E, n, k, tokens, TOPK, d1, ws.data_ptr(), nws, sp))

        st = torch.cuda.Stream(device=dev)
        with torch.cuda.stream(st):
            layer(0, st.cuda_stream)
            st.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=st):
                for i in range(NL):
                    layer(i, torch.cuda.current_stream().cuda_stream)
            g.replay()
            st.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            reps = 20
            e0.record(st)
            for _ in range(reps):
                g.replay()
            e1.record(st)
            st.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / (reps * NL)
        # the whole layer as FusedMoeGGUF::forward runs it: router + softmax + top-k, sort by expert, three grouped
        # matmuls (moe_gemm_gguf), silu(gate) * up, sum over top-k
        x3 = x.reshape(1, tokens, H)
        y = torch.empty((tokens, H), device=dev)
        with torch.cuda.stream(st):
            fused[0].forward(x3, tokens > 1, out=y)
            st.synchronize()
            g2 = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g2, stream=st):
                for i in range(NL):
                    fused[i].forward(x3, tokens > 1, out=y)
            g2.replay()
            st.synchronize()
            e0.record(st)
            for _ in range(reps):
                g2.replay()
            e1.record(st)
            st.synchronize()
        fused_us = e0.elapsed_time(e1) * 1e3 / (reps * NL)
        alg = distinct * 3 * 884736
        results.append({"tokens": tokens, "distinct_experts": distinct, "layer_us": round(us, 1), "algorithmic_MB": round(alg / 1e6, 1),
                        "GBps": round(alg / us / 1e3, 1), "tok_s_48_layers_expert_matmuls_only": round(tokens / (48 * us * 1e-6), 1),
                        "fused_moe_layer_us": round(fused_us, 1)})
    print(json.dumps({"metric": "Qwen3-30B-A3B-shape MoE layer, expert matmuls (Q4_K, 128 experts, top-8)", "unit": "us per layer", "n_gpus": 1,
                      "data": "synthetic", "config": {"workload": "gate + up [tokens, 2048] -> 768 and down [tokens*8, 768] -> 2048 via indexed_moe_forward, "
                                                                  "6 distinct layers rotated (2 GB), HIP graph; fused_moe_layer_us: the same "
                                                                  "layers through FusedMoeGGUF::forward (router, top-k, sort, moe_gemm_gguf x3, "
                                                                  "silu*up, sum over top-k)"},
                      "results": results}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--workload", choices=["decode", "prefill", "decode8b", "moe"], default="decode")
    ap.add_argument("--layers", type=int, default=32, help="--workload decode8b: number of decoder layers")
    ap.add_argument("--prompt", type=int, default=512, help="--workload decode8b: prompt tokens")
    ap.add_argument("--moe-tokens", default="1,16,256", help="--workload moe: token counts, comma separated")
    ap.add_argument("--wdtype", choices=sorted(WDTYPES), default="q4k",
                    help="weight format of --workload prefill / decode (the metric is quoted on q4k; other formats skip the 8B decoder and the CPU baseline)")
    ap.add_argument("--n", type=int, default=14336)
    ap.add_argument("--k", type=int, default=4096)
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--pool-mb", type=int, default=1280, help="distinct weight bytes rotated through (MB)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--pmc-mode", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="skip the labelled context numbers (cache-resident, pre-quantized)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (every configuration of the metric is single-GPU); use --gpus 1")
    if args.workload == "decode8b":
        print(json.dumps(decode8b(args)))
        return
    if args.workload == "moe":
        return moe(args)
    if args.steps is None:
        args.steps = 4000 if args.workload == "decode" else 50
    if args.warmup is None:
        args.warmup = 400 if args.workload == "decode" else 5
    if args.workload == "prefill":
        return prefill(args)

    import torch

    from candle_amd import _lib

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    L = _lib.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    n, k, m = args.n, args.k, args.batch
    WDT, w_ts, w_bs = WDTYPES[args.wdtype]
    fmt = FMT_NAMES[args.wdtype]
    headline = args.wdtype == "q4k"
    if not headline:
        args.no_cpu_baseline = True
    wbytes = L.cq_storage_bytes(WDT, n * k)
    alg_bytes = algorithmic_bytes(n, k, m, w_ts, w_bs)

    # ---- synthetic inputs, resident in HBM --------------------------------------------------
    pool = max(2, (args.pool_mb * 1000 * 1000 + wbytes - 1) // wbytes)
    if args.pmc_mode:
        pool = 8
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)
    weights = []
    for i in range(pool):
        wf = torch.randn((n, k), generator=gen, device=dev, dtype=torch.float32) * 0.02
        wq = torch.empty(wbytes, dtype=torch.uint8, device=dev)
        _lib.check("cq_quantize", L.cq_quantize(WDT, wf.data_ptr(), wq.data_ptr(), n * k, None))
        weights.append(wq)
        del wf
    x = torch.randn((m, k), generator=gen, device=dev, dtype=torch.float32)
    dst = torch.empty((m, n), dtype=torch.float32, device=dev)
    ws_bytes = L.cq_qmatmul_workspace_bytes(WDT, m, k, n)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    torch.cuda.synchronize()

    stream = torch.cuda.Stream(device=dev)

    def step(i, sp):
        """QMatMul::forward: activation quantization + matvec in one kernel."""
        _lib.check("cq_qmatmul_forward", L.cq_qmatmul_forward(WDT, weights[i % pool].data_ptr(), x.data_ptr(), 0, dst.data_ptr(), 0,
                                                              m, k, n, ws.data_ptr(), ws_bytes, sp))

    def matvec_prequantized(i, sp):
        _lib.check("cq_matvec", L.cq_matvec(WDT, weights[i % pool].data_ptr(), ws.data_ptr(), dst.data_ptr(), 0, k, n, m, n, sp))

    if args.pmc_mode:
        # plain launches (one dispatch row per kernel in the counter CSV) + a copy of known size
        with torch.cuda.stream(stream):
            for i in range(2 * pool):
                step(i, stream.cuda_stream)
            a = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
            b = torch.empty_like(a)
            stream.synchronize()
            for _ in range(4):
                b.copy_(a)
        torch.cuda.synchronize()
        print(json.dumps({"pmc_mode": True, "copy_bytes": 256 << 20, "step_algorithmic_bytes": alg_bytes}))
        return

    # The step is a few microseconds of GPU work: capture one rotation over the pool in a HIP graph
    # so that host launch latency is not what gets measured.
    def capture(fn, same_weight=False):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(stream):
            fn(0, stream.cuda_stream)          # warm the code path before capture
            stream.synchronize()
            with torch.cuda.graph(g, stream=stream):
                sp = torch.cuda.current_stream().cuda_stream
                for i in range(pool):
                    fn(0 if same_weight else i, sp)
        return g

    def run(graph, steps):
        reps = max(1, (steps + pool - 1) // pool)
        with torch.cuda.stream(stream):
            for _ in range(reps):
                graph.replay()
        return reps * pool

    def event_us(graph, steps):
        run(graph, args.warmup)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        with torch.cuda.stream(stream):
            e0.record(stream)
            done = run(graph, steps)
            e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / done

    g_step = capture(step)

    # ---- timed region: K steps (rounded up to whole rotations of the pool), wall clock ------------
    run(g_step, args.warmup)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    done = run(g_step, args.steps)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / done
    value = alg_bytes / (ms_per_step * 1e-3) / 1e9

    # ---- dominant kernel (the step IS one kernel): HIP events around the same back-to-back launches ----
    kern_us = event_us(g_step, args.steps)
    achieved = alg_bytes / (kern_us * 1e-6) / 1e9
    # context numbers, labelled: the same kernel with the weights resident in the Infinity Cache (one
    # tensor reused), and the matvec over activations quantized beforehand by cq_quantize_act
    extra = None
    if not args.no_extra:
        resident_us = event_us(capture(step, same_weight=True), args.steps)
        _lib.check("cq_quantize_act", L.cq_quantize_act(WDT, x.data_ptr(), 0, ws.data_ptr(), k, m, None))
        torch.cuda.synchronize()
        preq_us = event_us(capture(matvec_prequantized), args.steps)
        # the yardstick: a kernel that only reads the same rotated tensors, same launch shape
        sink = torch.zeros(4, dtype=torch.int32, device=dev)
        read_bytes = wbytes - wbytes % 16

        def plain_read(i, sp):
            _lib.check("cq_bench_read", L.cq_bench_read(weights[i % pool].data_ptr(), read_bytes, sink.data_ptr(), sp))

        read_us = event_us(capture(plain_read), args.steps)
        extra = {"plain_read_us": round(read_us, 3), "plain_read_GBps": round(read_bytes / (read_us * 1e-6) / 1e9, 1),
                 "infinity_cache_resident_us": round(resident_us, 3),
                 "infinity_cache_resident_GBps": round(alg_bytes / (resident_us * 1e-6) / 1e9, 1),
                 "prequantized_matvec_us": round(preq_us, 3),
                 "prequantized_matvec_GBps": round(alg_bytes / (preq_us * 1e-6) / 1e9, 1)}

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
                           % ("Q8_K" if w_bs == 256 else "Q8_0"),
                   "n": n, "k": k, "batch": m},
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "roofline": {"bound": "hbm", "kernel": "qmv_kernel<%s, NB=%d, fused f32 activations>" % (fmt, m), "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": committed_traffic() if headline else None,
                     "avg_kernel_us": round(kern_us, 3), "algorithmic_bytes_per_launch": alg_bytes},
        "extra": extra,
    }

    if not args.no_extra and headline:
        # the second half of the metric: the 8B-shape decoder (same protocol as --workload decode8b)
        d8 = argparse.Namespace(layers=32, prompt=512, steps=256)
        r = decode8b(d8)
        out["decode_8b"] = {"tok_s": r["value"], "ms_per_token": r["ms_per_step"], "prompt_tok_s": r["prompt_tok_s"],
                            "frac_of_roofline_tok_s": r["roofline"]["frac_of_roofline_tok_s"],
                            "roofline_tok_s": r["roofline"]["roofline_tok_s_weights_only"],
                            "weight_bytes_per_token": r["weight_bytes_per_token"], "workload": r["config"]["workload"]}

    if not args.no_cpu_baseline:
        import oracle
        cores = min(len(os.sched_getaffinity(0)), int(os.environ.get("OMP_NUM_THREADS", "16")), 16)
        host_pool = min(pool, 8)
        hw = [weights[i].cpu().numpy() for i in range(host_pool)]
        hx = x.cpu().numpy()
        oracle.matmul_fast(Q4K, hx, hw[0], n, cores)
        t0 = time.perf_counter()
        it = 0
        while time.perf_counter() - t0 < args.cpu_seconds:
            oracle.matmul_fast(Q4K, hx, hw[it % host_pool], n, cores)
            it += 1
        dt = (time.perf_counter() - t0) / it
        out["cpu_baseline"] = {"value": round(alg_bytes / dt / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
                               "sample": "%d calls of the same 1x%d->%d Q4_K matvec over %d rotated host weight copies (%.1f s); "
                                         "C restatement of candle's CPU path: Q8_K activation quantize + AVX2 vec_dot + column split over threads"
                                         % (it, k, n, host_pool, args.cpu_seconds),
                               "ms_per_call": round(dt * 1e3, 4)}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
