#!/usr/bin/env python3
"""Benchmark of the quantized MoE layer on one MI355X.

The default run measures both halves of the metric on the Qwen3-30B-A3B-shaped layer (hidden 2048,
128 experts, top-8 renormalised, intermediate 768, 4-bit g64):
  * decode, batches 1 / 8 / 32 -- the headline `value` is tokens/s at batch 32, `roofline` prices the
    dominant kernel of that step against the HBM peak;
  * prefill, 4096 tokens with a Zipf(1.1) router bias -- `roofline_prefill` prices its dominant kernel
    against the dense bf16 MFMA peak, `prefill` holds tokens/s and the layer-level fraction.
A "step" is one forward of the layer over one batch whose inputs are already in HBM.  Steps rotate
over several distinct weight sets whose total size exceeds the 256 MB Infinity Cache, so weights
stream from HBM every step.

Kernel durations are the ones mi_moe_forward_timed reports from each dispatch's own start and end
time stamps (what rocprofv3 lists as the kernel's duration), averaged over the timed steps.

Prints ONE JSON line (see --help for the other workloads).  The CPU-baseline leg times the CPU
oracle (a restatement of the MLX CPU op sequence; MLX itself is not available) on the host cores;
it is the only part of this script that touches oracle/.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0       # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
# HBM bytes per launch of each workload's roofline kernel, from two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE)
# scaled by what the same counters read for a plain copy kernel of known size.  Counters cannot be read from
# inside this script: the figure is carried from the named file under profiles/, it is not measured by this run.
CARRIED_TRAFFIC = {
    "decode": (1.975e8, "profiles/qmm_small_kernel_decode_batch32_hbm_traffic.txt"),
    "prefill": (4.054e8, "profiles/qmm_large_kernel_prefill_tokens4096_counters.txt"),
    "mixtral_decode": (2.528e8, "profiles/qmm_small_kernel_decode_mixtral_batch1.txt"),
}

WORKLOADS = {
    # name: (config key, batches, headline batch, zipf s, bound)
    "decode": ("qwen3_30b_a3b", [1, 8, 32], 32, None, "hbm"),
    "decode_batch1": ("qwen3_30b_a3b", [1], 1, None, "hbm"),   # one batch per process: for per-kernel profiles
    "decode_batch8": ("qwen3_30b_a3b", [8], 8, None, "hbm"),
    "prefill": ("qwen3_30b_a3b", [4096], 4096, 1.1, "mfma"),
    "mixtral_decode": ("mixtral_8x7b", [1], 1, None, "hbm"),
    "mixtral_prefill": ("mixtral_8x7b", [2048], 2048, None, "mfma"),
    "qwen3_235b_prefill": ("qwen3_235b_a22b", [8192], 8192, 1.3, "mfma"),
    "tiny": ("tiny", [32], 32, None, "hbm"),
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="default", choices=["default"] + sorted(WORKLOADS),
                    help="default = decode (headline) followed by prefill, both in the one JSON line")
    ap.add_argument("--layers", type=int, default=0, help="distinct weight sets to rotate over (0 = auto)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--serial-kernels", action="store_true",
                    help="every step through mi_moe_forward_timed: kernels run one after the other on one stream "
                         "(for per-kernel profiles; a prefill-sized mi_moe_forward runs four chains side by side)")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--only-headline", action="store_true", help="run only the headline batch of the workload")
    ap.add_argument("--batches", default="", help="comma-separated batch sizes to run besides the headline batch")
    ap.add_argument("--copy-probe", type=int, default=0,
                    help="first launch N plain 256 MiB copy kernels (a known-size reference for profiler counters)")
    return ap.parse_args()


def time_steps(fn, steps, warmup, torch):
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        fn(warmup + i)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps * 1e3


def tile_class_rows(counts, cfg, T, capi):
    """Rows of the batch that each grouped-product kernel processes: [256-row tiles, 128-row tiles,
    64-row tiles, streamed], by the library's own rule (capi.tile_rule, capi.segment_rows_by_kernel)."""
    tiled, tmr = capi.tile_rule(cfg.c_struct(), T)
    rows = [0, 0, 0, 0]
    for c in counts:
        rows = [a + b for a, b in zip(rows, capi.segment_rows_by_kernel(c, tiled, tmr))]
    return rows


def run_workload(name, args, torch, m, synth, dev):
    """Times one workload; returns a dict with the headline step, the per-batch detail and what the
    roofline block needs."""
    cfg_name, batches, headline, zipf_s, bound = WORKLOADS[name]
    if args.only_headline:
        batches = [headline]
    if args.batches and args.workload != "default":
        batches = sorted(set(int(b) for b in args.batches.split(",")) | {headline})
    cfg = synth.CONFIGS[cfg_name]
    layer_bytes = synth.layer_bytes_per_expert(cfg) * cfg.n_experts
    n_layers = args.layers or max(2, min(8, int(1.4e9 // layer_bytes) + 1))
    if layer_bytes > 1.0e9:
        n_layers = args.layers or 2
    steps, warmup = args.steps, args.warmup
    if bound == "mfma" and args.workload == "default":
        steps, warmup = max(10, steps // 4), max(2, warmup // 4)  # a prefill step is 7 times a decode step
    blocks = [synth.make_block(cfg, seed=args.seed + 31 * i, device=dev, zipf_s=zipf_s, gen_device="cuda")
              for i in range(n_layers)]
    torch.cuda.synchronize()

    detail = {}
    head = None
    for T in batches:
        x = synth.make_tokens(cfg, T, seed=args.seed, device=dev)
        outs = [torch.empty_like(x) for _ in range(n_layers)]
        for b in blocks:
            b.reserve(T)
        # realised routing (per weight set)
        actives, counts_stats, class_rows = [], [], []
        for b in blocks:
            _, dbg = b.forward(x, debug=True)
            c = dbg["counts"].cpu().numpy()
            actives.append(int((c > 0).sum()))
            counts_stats.append((int(c.max()), float(c.mean()), int(c.min())))
            class_rows.append(tile_class_rows(c, cfg, T, m.capi))
        n_active = sum(actives) / len(actives)
        class_rows = [sum(r[i] for r in class_rows) / len(class_rows) for i in range(4)]

        if args.serial_kernels:
            step_fn = lambda blk, xx, oo: blk.forward_timed(xx, out=oo)
        else:
            step_fn = lambda blk, xx, oo: blk.forward(xx, out=oo)
        graph = None
        if not args.no_graph and not args.serial_kernels:
            # one graph replays a forward through every weight set (launch overhead amortised the
            # way a serving loop would capture a whole decode step)
            s = torch.cuda.Stream()
            s.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(s):
                for i, b in enumerate(blocks):
                    b.forward(x, out=outs[i])
            torch.cuda.current_stream().wait_stream(s)
            torch.cuda.synchronize()
            # (several passes over the weight sets per graph while a step is short: a replay's own cost is
            # shared by more steps)
            passes = max(1, min(4, steps // (4 * n_layers))) if bound == "hbm" else 1
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for _ in range(passes):
                    for i, b in enumerate(blocks):
                        b.forward(x, out=outs[i])
            eager_ref = [o.clone() for o in outs]
            graph.replay()
            torch.cuda.synchronize()
            for o, r in zip(outs, eager_ref):
                assert torch.equal(o, r), "graph replay differs from the eager result"

        if graph is not None:
            # a step = one forward; one replay = n_layers steps
            per_replay = n_layers * passes
            reps = max(1, steps // per_replay)
            wreps = max(1, warmup // per_replay)
            graph_ms = time_steps(lambda i: graph.replay(), reps, wreps, torch) / per_replay
            graph_steps = reps * per_replay
        eager_ms = time_steps(lambda i: step_fn(blocks[i % n_layers], x, outs[i % n_layers]), steps, warmup, torch)
        # the step that is reported: the faster of the two ways to launch the same forwards (a replayed graph
        # saves host work per launch, but a forward that forks its kernel chains over streams pays for every
        # fork and join in a replay); both figures stay in the detail
        if graph is not None and graph_ms <= eager_ms:
            ms, steps_done, launch = graph_ms, graph_steps, "hip-graph"
        else:
            ms, steps_done = eager_ms, steps
            launch = "eager, one kernel at a time" if args.serial_kernels else "eager"

        # spread of single steps (event pair around each eager step) and the cache-resident figure
        # (one weight set only: at decode sizes it stays in the 256 MB Infinity Cache)
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        for i, (e0, e1) in enumerate(evs):
            e0.record()
            step_fn(blocks[i % n_layers], x, outs[i % n_layers])
            e1.record()
        torch.cuda.synchronize()
        per_step = sorted(e0.elapsed_time(e1) for e0, e1 in evs)
        pct = lambda q: per_step[min(len(per_step) - 1, int(q * len(per_step)))]
        resident_ms = time_steps(lambda i: step_fn(blocks[0], x, outs[0]), steps, warmup, torch)

        # per-stage times (events between the stages) and the grouped-product kernels' own durations
        # (time stamps of each dispatch), same number of steps
        stage = [0.0] * m.capi.N_STAGES
        kern = [0.0] * m.capi.N_KERNEL_TIMES
        for i in range(steps):
            _, st, km = blocks[i % n_layers].forward_timed(x, out=outs[i % n_layers], kernels=True)
            stage = [a + b for a, b in zip(stage, st)]
            kern = [a + b for a, b in zip(kern, km)]
        stage = [v / steps for v in stage]
        kern = [v / steps for v in kern]

        P = T * cfg.top_k
        qbytes = lambda n, k: n * k * cfg.bits // 8 + (n * k // cfg.group_size) * 4
        gu_bytes = n_active * 2 * qbytes(cfg.intermediate, cfg.hidden) + T * cfg.hidden * 2 + P * cfg.intermediate * 2
        dn_bytes = n_active * qbytes(cfg.hidden, cfg.intermediate) + P * cfg.intermediate * 2 + P * cfg.hidden * 2
        alg_bytes = synth.decode_algorithmic_bytes(cfg, T, n_active)
        flops = synth.prefill_flops(cfg, T)
        gu_flops = P * 2 * 2 * cfg.hidden * cfg.intermediate
        gu_kernel_ms, dn_kernel_ms = sum(kern[0:4]), sum(kern[4:8])
        detail[str(T)] = {
            "tokens_per_s": T / (ms * 1e-3), "ms_per_step": ms, "launch": launch,
            "ms_per_step_graph_replay": graph_ms if graph is not None else None, "ms_per_step_eager": eager_ms,
            "steps": steps_done, "active_experts": n_active,
            "step_ms_p10_p50_p90_event_timed": [round(pct(0.1), 5), round(pct(0.5), 5), round(pct(0.9), 5)],
            "ms_per_step_cache_resident_single_weight_set": resident_ms,
            "counts_max_mean_min": counts_stats[0],
            "layer_algorithmic_MB": alg_bytes / 1e6, "layer_GBps": alg_bytes / (ms * 1e-3) / 1e9,
            "layer_hbm_frac": alg_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            "layer_TFLOPs": flops / (ms * 1e-3) / 1e12,
            "layer_mfma_frac": flops / (ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
            "stage_us_between_events": {n: round(v * 1e3, 2) for n, v in zip(m.capi.STAGE_NAMES, stage)},
            "kernel_us": {n: round(v * 1e3, 2) for n, v in zip(m.capi.KERNEL_NAMES, kern) if v > 0},
            "rows_per_kernel_class": dict(zip(("tiles256", "tiles128", "tiles64", "streamed"), class_rows)),
            "gate_up_GBps": gu_bytes / (gu_kernel_ms * 1e-3) / 1e9 if gu_kernel_ms else None,
            "down_GBps": dn_bytes / (dn_kernel_ms * 1e-3) / 1e9 if dn_kernel_ms else None,
            "gate_up_TFLOPs": gu_flops / (gu_kernel_ms * 1e-3) / 1e12 if gu_kernel_ms else None,
            "gate_up_mfma_frac": gu_flops / (gu_kernel_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS if gu_kernel_ms else None,
        }
        if T == headline:
            head = dict(stage_ms=stage, ms=ms, launch=launch, T=T, gu_bytes=gu_bytes, dn_bytes=dn_bytes, gu_flops=gu_flops, steps=steps_done, warmup=warmup, kern=kern,
                        class_rows=class_rows, per_row_gu_flops=2 * 2 * cfg.hidden * cfg.intermediate)
        del outs, graph

    traffic, traffic_src = CARRIED_TRAFFIC.get(name, (None, None))
    if bound == "hbm":
        # the streamed gate/up + SwiGLU kernel: every segment streams at decode sizes
        k_ms, k_bytes = head["kern"][3], head["gu_bytes"]
        k_name = "qmm_small_kernel (gate/up + SwiGLU, streamed)"
        achieved = k_bytes / (k_ms * 1e-3) / 1e9
        roofline = {"kernel": k_name, "bound": "hbm", "achieved": achieved,
                    "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS,
                    "traffic": traffic, "traffic_source": traffic_src and traffic_src + " (carried, not measured by this run)",
                    "algorithmic_bytes_per_launch": head["gu_bytes"], "kernel_us": k_ms * 1e3,
                    "kernel_us_source": "start/end time stamps of the dispatch (hipExtLaunchKernelGGL events), mean over the timed steps "
                                        "(mi_moe_forward_timed: same kernels, same order and stream as mi_moe_forward at decode sizes)",
                    "stream_probe": stream_probe(m, head["gu_bytes"], dev)}
    else:
        # the dominant kernel: the tile class that holds most rows (256-row tiles at prefill sizes)
        cls = max(range(3), key=lambda i: head["class_rows"][i])
        k_ms, k_rows = head["kern"][cls], head["class_rows"][cls]
        k_name = "qmm_large_kernel (gate/up + SwiGLU, %d-row tiles)" % (256, 128, 64)[cls]
        k_flops = k_rows * head["per_row_gu_flops"]
        achieved = k_flops / (k_ms * 1e-3) / 1e12
        roofline = {"kernel": k_name, "bound": "mfma",
                    "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                    "frac": achieved / MFMA_BF16_PEAK_TFLOPS,
                    "traffic": traffic, "traffic_source": traffic_src and traffic_src + " (carried, not measured by this run)",
                    "algorithmic_flops_per_launch": k_flops, "rows_per_launch": k_rows,
                    "kernel_us": k_ms * 1e3,
                    "kernel_us_source": "start/end time stamps of the dispatch (hipExtLaunchKernelGGL events), mean over the timed steps, "
                                        "kernels launched one after the other on one stream (mi_moe_forward_timed); the timed step itself "
                                        "(ms_per_step) runs mi_moe_forward's own schedule, tile classes side by side on two to four streams",
                    "serial_kernels_us_sum_vs_step_us": [round((sum(head["kern"]) + sum(head["stage_ms"][i] for i in (0, 1, 2, 5))) * 1e3, 1),
                                                         round(head["ms"] * 1e3, 1)],
                    "dense_gemm_yardstick": dense_gemm_yardstick(torch, int(round(k_rows)), 2 * cfg.intermediate, cfg.hidden, dev),
                    "gate_up_stage": {"flops": head["gu_flops"], "kernels_us": sum(head["kern"][0:4]) * 1e3,
                                      "TFLOPs": head["gu_flops"] / (sum(head["kern"][0:4]) * 1e-3) / 1e12,
                                      "frac": head["gu_flops"] / (sum(head["kern"][0:4]) * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS}}
    workload = "%s %s-bit g64 MoE layer, %s, batch %d" % (cfg_name, cfg.bits, name, headline)
    config = {"workload": workload, "hidden": cfg.hidden, "n_experts": cfg.n_experts, "top_k": cfg.top_k,
              "intermediate": cfg.intermediate, "bits": cfg.bits, "batch": headline, "weight_sets_rotated": n_layers,
              "zipf_s": zipf_s,
              "launch": head["launch"]}
    return dict(cfg=cfg, blocks=blocks, head=head, headline=headline, detail=detail, roofline=roofline, bound=bound,
                config=config)


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    import torch
    import mlx_rs_amd as m
    from mlx_rs_amd import synth

    m.load_library()  # raises if the HIP library is missing
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = "cuda:0"
    torch.cuda.set_device(0)
    if args.copy_probe:
        # an elementwise kernel that reads 256 MiB and writes 256 MiB
        src = torch.zeros(64 << 20, dtype=torch.int32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(args.copy_probe):
            torch.add(src, 1, out=dst)
        torch.cuda.synchronize()
        del src, dst

    first = "decode" if args.workload == "default" else args.workload
    w = run_workload(first, args, torch, m, synth, dev)
    head, bound = w["head"], w["bound"]
    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline(w["cfg"], w["blocks"][0], w["headline"], args.seed, synth)
    out = {
        "metric": "MoE-layer tokens/sec (%s)" % ("decode" if bound == "hbm" else "prefill"),
        "value": w["headline"] / (head["ms"] * 1e-3), "unit": "tokens/s", "n_gpus": 1,
        "steps": head["steps"], "warmup": head["warmup"], "ms_per_step": head["ms"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic", "config": w["config"],
        "layer_frac_of_peak": w["detail"][str(w["headline"])]["layer_hbm_frac" if bound == "hbm" else "layer_mfma_frac"],
        "roofline": w["roofline"], "cpu_baseline": cpu, "detail": w["detail"],
    }
    if args.workload == "default":
        del w  # the decode weight sets go before the prefill ones are built
        torch.cuda.empty_cache()
        p = run_workload("prefill", args, torch, m, synth, dev)
        d = p["detail"][str(p["headline"])]
        out["roofline_prefill"] = p["roofline"]
        out["prefill"] = {"metric": "MoE-layer tokens/sec (prefill)", "value": d["tokens_per_s"], "unit": "tokens/s",
                          "ms_per_step": d["ms_per_step"], "steps": d["steps"], "config": p["config"],
                          "layer_TFLOPs": d["layer_TFLOPs"], "layer_frac_of_peak": d["layer_mfma_frac"], "detail": d}
    print(json.dumps(out))


def dense_gemm_yardstick(torch, M, N, K, dev):
    """A library dense bf16 GEMM of the roofline kernel's aggregate shape (M rows of the dominant tile class,
    N = gate + up columns, K = hidden), timed the same way: what torch.matmul (hipBLASLt / rocBLAS) reaches
    on this box for [M, K] x [K, N].  A yardstick beside the vendor peak, not on the product path: the
    product kernel also unpacks 4-bit codes, gathers its rows and applies SwiGLU."""
    a = torch.randn((M, K), device=dev, dtype=torch.bfloat16)
    b = torch.randn((N, K), device=dev, dtype=torch.bfloat16)
    out = torch.empty((M, N), device=dev, dtype=torch.bfloat16)
    for _ in range(5):
        torch.matmul(a, b.t(), out=out)
    torch.cuda.synchronize()
    reps = 30
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        torch.matmul(a, b.t(), out=out)
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) / reps * 1e3
    tf = 2.0 * M * N * K / (us * 1e-6) / 1e12
    return {"what": "torch.matmul bf16 [%d, %d] x [%d, %d]^T, yardstick only (not on the product path)" % (M, K, N, K),
            "us": us, "TFLOPs": tf, "frac_of_peak": tf / MFMA_BF16_PEAK_TFLOPS}


def stream_probe(m, nbytes, dev):
    """What a launch of the roofline kernel's size can pull from HBM on this box: the library's bare
    streaming kernel (the product kernel's access shape, nothing else) over as many bytes as the
    gate/up launch reads, launched back to back over 12 distinct regions (cold in every cache)."""
    import torch
    lib = m.capi.load_library()
    size = max(32768, int(nbytes) // 32768 * 32768)
    regions = 12
    buf = torch.ones(regions * size, dtype=torch.uint8, device=dev)
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    def launch(i):
        m.capi.check(lib.mi_moe_stream_probe(buf.data_ptr() + (i % regions) * size, size, sink.data_ptr(), st))
    for i in range(regions):
        launch(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    reps = 4 * regions
    e0.record()
    for i in range(reps):
        launch(i)
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) / reps * 1e3
    return {"bytes": size, "us_per_launch": us, "GBps": size / (us * 1e-6) / 1e9,
            "frac_of_peak": size / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS}


def cpu_baseline(cfg, block, T, seed, synth):
    """Times the CPU oracle (op-by-op 'strict' mode: the MLX CPU op sequence restated) on the
    host cores for the same layer and batch; a bounded sample (a few repeats, or a token
    subsample for the large prefill shapes)."""
    import numpy as np
    import oracle
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from helpers import bits_u16, bits_u32

    threads = min(16, len(os.sched_getaffinity(0)))
    W = dict(router_w=bits_u16(block.gate_weight),
             router_bias=None if block.router_bias is None else block.router_bias.cpu().numpy(),
             gate=(bits_u32(block.gate_proj.weight), bits_u16(block.gate_proj.scales), bits_u16(block.gate_proj.biases)),
             up=(bits_u32(block.up_proj.weight), bits_u16(block.up_proj.scales), bits_u16(block.up_proj.biases)),
             down=(bits_u32(block.down_proj.weight), bits_u16(block.down_proj.scales), bits_u16(block.down_proj.biases)))
    Ts = min(T, 256)
    x = bits_u16(synth.make_tokens(cfg, Ts, seed=seed, device="cpu"))
    ocfg = oracle.make_config(cfg.hidden, cfg.n_experts, cfg.top_k, cfg.intermediate, cfg.bits, cfg.group_size,
                              cfg.score_mode)
    oracle.moe_forward(ocfg, W, x, strict=True, n_threads=threads, debug=False)  # warm-up
    times = []
    t_all = time.perf_counter()
    while len(times) < 5 or (time.perf_counter() - t_all < 10.0 and len(times) < 50):
        t0 = time.perf_counter()
        oracle.moe_forward(ocfg, W, x, strict=True, n_threads=threads, debug=False)
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    t1 = []
    for _ in range(2):  # the same layer on one thread
        t0 = time.perf_counter()
        oracle.moe_forward(ocfg, W, x, strict=True, n_threads=1, debug=False)
        t1.append(time.perf_counter() - t0)
    model = "unknown CPU"
    try:
        with open("/proc/cpuinfo") as f:
            model = next(l.split(":", 1)[1].strip() for l in f if l.startswith("model name"))
    except (OSError, StopIteration):
        pass
    sample = "%d runs of the full layer at batch %d" % (len(times), Ts)
    if Ts != T:
        sample += " (token subsample of the %d-token workload; tokens/s is per token, so no scaling applied)" % T
    return {"value": Ts / med, "unit": "tokens/s", "cores": threads, "kind": "port",
            "sample": sample + "; CPU oracle in op-by-op mode (restatement of the MLX CPU op sequence; MLX itself "
                               "cannot be built offline), OpenMP",
            "cpu_model": model, "single_thread_tokens_per_s": Ts / min(t1)}


if __name__ == "__main__":
    main()
