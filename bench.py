#!/usr/bin/env python3
"""Benchmark of the MoE hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one pass of the layer over one batch already resident in HBM:
softmax top-k router -> zbal_fused_deep_moe (permute + fp8 quantise, grouped
GEMM 1 with SwiGLU + requantise, grouped GEMM 2, weighted combine), all through
the zbal C ABI. The workload is the DeepSeek-V3-style prefill share: 4096
tokens x hidden 7168, 32 local experts, top-8 over uniform-random logits, fp8
e4m3 with 1x128 activation and 128x128 weight scales, intermediate 2048.
Synthetic data, random weights. The default run measures the headline workload
and then, under `other_workloads` of the same JSON line, the other
configurations the metric names: the 8 x 256 MiB local reduction (bf16 and
fp32), the 128-token W8A8 decode layer with Zipf(1.2) expert popularity and the
16384-token W4A8 layer. `--workload decode | qwen_w4a8 | reduce` measures one of
them alone, with the full line.

No cache flush between steps: one step streams 1.4 GB of weights and 0.9 GB of
activations through a 32-MiB L2 and a 256-MiB memory-side cache, so every step
starts cold (`config.l2_flush_between_steps` says so in the line).

Prints ONE JSON line. `value` is tokens/s of the whole step. `roofline`
prices the dominant kernel (grouped GEMM 1) from its algorithmic FLOPs and
its average duration measured with HIP events in a second loop that issues
the same stages one by one through the inner kernel ABI. `cpu_baseline` is
the CPU oracle (a scalar C++ restatement, OpenMP over rows) timed on the
host on a bounded sample of the same batch; the same sample is used to check
the GPU result.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP8_TFLOPS = 5000.0      # MI355X dense fp8 MFMA
PEAK_HBM_GBS = 8000.0         # MI355X HBM3E


def measured_traffic(key):
    """HBM bytes per launch of the dominant kernel of workload `key`, or None: 2.0 x FETCH_SIZE + 1.0 x WRITE_SIZE from
    two `rocprofv3 --pmc` runs of this script, written to profiles/traffic.json together with the profile summaries
    that show the counters and their calibration (the file names the summary of every entry)."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            entry = json.load(f).get(key)
        return None if entry is None else float(entry["bytes_per_launch"])
    except (OSError, ValueError, KeyError, TypeError):
        return None



def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--tokens", type=int, default=4096, help="development only; the reported workload is 4096")
    ap.add_argument("--cpu-sample-tokens", type=int, default=2560)
    ap.add_argument("--workload", choices=["prefill", "prefill_w8a8", "decode", "qwen_w4a8", "reduce"], default="prefill",
                    help="prefill = the headline fp8 MoE layer (default); prefill_w8a8 = the same shape in W8A8 (profiling: no "
                         "BASELINE configuration); decode = 128-token W8A8 layer with Zipf routing; qwen_w4a8 = 16384-token "
                         "W4A8 layer; reduce = the 8 x 256 MiB local reduction")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--equal-rows", action="store_true",
                    help="profiling only (prefill): token t picks experts (t*topk + j) mod experts, so every expert receives "
                         "exactly tokens*topk/experts rows; the figure says what the ragged row counts of random routing cost")
    ap.add_argument("--no-others", action="store_true",
                    help="headline workload only: leave out the `other_workloads` block (reduce, decode, W4A8)")
    return ap.parse_args()


def main():
    args = parse()
    if args.gpus != 1:
        sys.stderr.write("bench.py: this build measures one GPU's share of the path; runs with --gpus > 1 are not "
                         "part of it (no collectives, no sharding). Use --gpus 1.\n")
        sys.exit(2)

    import numpy as np
    import torch
    from memfabric_hybrid_amd import capi
    from memfabric_hybrid_amd.operators import OperatorBuffer as Buffer

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    dev = torch.device("cuda", 0)
    buf = Buffer()
    lib = buf.lib
    if args.workload == "reduce":
        line = bench_reduce(args, torch, np, capi, buf)
    else:
        line = bench_moe(args, torch, np, capi, buf, args.workload)
        if args.workload == "prefill" and not args.no_others and args.tokens == 4096:
            # the rest of the metric (reduce % HBM, the decode and W4A8 layers), measured in the same run
            line["other_workloads"] = other_workloads(args, torch, np, capi, buf)
    print(json.dumps(line))
    buf.close()


def other_workloads(args, torch, np, capi, buf):
    """The configurations beside the headline one, each timed like it: `ms` per step, the dominant kernel's
    algorithmic rate against its roofline, and whether the result matched the CPU oracle."""
    out = []
    red = bench_reduce(args, torch, np, capi, buf)
    for name, v in red["variants"].items():
        out.append({"workload": "local reduce-scatter shard, 8 x 256 MiB %s (BASELINE configs[3])" % name, "ms": v["ms"],
                    "achieved": v["gbs"], "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": v["gbs"] / PEAK_HBM_GBS,
                    "exact": v["exact"]})
    torch.cuda.empty_cache()
    for wl in ("decode", "qwen_w4a8"):
        m = bench_moe(args, torch, np, capi, buf, wl)
        r = m["roofline"]
        out.append({"workload": m["config"]["workload"], "ms": m["ms_per_step"], "tokens_per_s": m["value"],
                    "kernel": r["kernel"], "achieved": r["achieved"], "peak": r["peak"], "unit": r["unit"], "frac": r["frac"],
                    "stages_ms": m["stages"]["ms"],
                    "exact": None if m["parity"] is None else m["parity"]["bit_exact"],
                    "parity_tokens": None if m["parity"] is None else m["parity"]["tokens"]})
        torch.cuda.empty_cache()
    return out


# mode: zbal_fused_deep_moe quantMode (1 = W8A8, 2 = fp8 block-scaled, 3 = W4A8)
MOE_WORKLOADS = {
    "prefill": dict(name="DeepSeek-V3-style prefill share (BASELINE configs[1])", T=4096, H=7168, E=32, K=8, I=2048,
                    mode=2, zipf=None, quant="fp8 e4m3, act 1x128, weight 128x128", dtype="fp8_e4m3"),
    "prefill_w8a8": dict(name="the prefill share's shape in W8A8 (profiling; not a BASELINE configuration)", T=4096, H=7168, E=32,
                         K=8, I=2048, mode=1, zipf=None, quant="W8A8 int8, per-token act, per-channel weight scales",
                         dtype="int8"),
    "decode": dict(name="low-latency decode share (BASELINE configs[2])", T=128, H=7168, E=32, K=8, I=2048,
                   mode=1, zipf=1.2, quant="W8A8 int8, per-token act, per-channel weight scales", dtype="int8"),
    "qwen_w4a8": dict(name="Qwen3-MoE-style W4A8 layer (BASELINE configs[4])", T=16384, H=4096, E=128, K=8, I=1536,
                      mode=3, zipf=None, quant="W4A8: int8 per-token act, int4 g128 weights, fp16 group scales",
                      dtype="int8"),
}


def make_weights(torch, buf, dev, mode, E, k, n):
    """Random expert weights [E, k, n] in the logical layout, their pre-packed form and scales for `mode`."""
    if mode == 2:
        w = torch.empty((E, k, n), device=dev, dtype=torch.float8_e4m3fn)
        for e in range(E):
            w[e] = (torch.randn((k, n), device=dev) * 100.0).clamp_(-448, 448).to(torch.float8_e4m3fn)
        s = (torch.rand((E, k // 128, n // 128), device=dev) + 0.5) * (1.0 / (100.0 * k ** 0.5))
        return w, buf.prepack_weight(w), s
    if mode == 1:
        w = torch.randint(-127, 128, (E, k, n), device=dev, dtype=torch.int8)
        s = (torch.rand((E, n), device=dev) + 0.5) * (1.0 / (73.0 * k ** 0.5))
        return w, buf.prepack_weight(w), s
    w = torch.randint(-8, 8, (E, k, n), device=dev, dtype=torch.int8)
    s = ((torch.rand((E, k // 128, n), device=dev) + 0.5) * (1.0 / (4.6 * k ** 0.5))).to(torch.float16)
    return w, buf.prepack_weight(w, int4=True), s


def bench_moe(args, torch, np, capi, buf, workload):
    cfg = MOE_WORKLOADS[workload]
    lib = buf.lib
    dev = torch.device("cuda", 0)
    T = args.tokens if workload == "prefill" else cfg["T"]
    H, E, K, I, mode = cfg["H"], cfg["E"], cfg["K"], cfg["I"], cfg["mode"]
    N1 = 2 * I
    rows = T * K
    torch.manual_seed(0)
    x = torch.randn((T, H), device=dev, dtype=torch.float32).to(torch.bfloat16)
    if workload == "prefill" and args.equal_rows:
        picks = (torch.arange(T, device=dev)[:, None] * K + torch.arange(K, device=dev)[None, :]) % E
        logits = torch.rand((T, E), device=dev, dtype=torch.float32)
        logits.scatter_add_(1, picks, torch.ones((T, K), device=dev))
    elif cfg["zipf"] is None:
        logits = torch.rand((T, E), device=dev, dtype=torch.float32)          # uniform-random logits
    else:
        # Zipf(s) popularity over a fixed random permutation of the experts; adding Gumbel noise to log p makes
        # the router's top-k a draw of K distinct experts with those popularities
        p = 1.0 / torch.arange(1, E + 1, device=dev, dtype=torch.float32) ** cfg["zipf"]
        p = p[torch.randperm(E, device=dev)]
        u = torch.rand((T, E), device=dev).clamp_(1e-9, 1 - 1e-9)
        logits = (torch.log(p / p.sum())[None, :] - torch.log(-torch.log(u))).contiguous()

    w1_logical, w1, s1 = make_weights(torch, buf, dev, mode, E, H, N1)       # logical = [E, K, N] of the operator API
    w2_logical, w2, s2 = make_weights(torch, buf, dev, mode, E, I, H)
    if mode == 1:
        s2 = s2.to(torch.bfloat16)                                           # the reference's GMM2 scale type
    torch.cuda.synchronize()

    ws = torch.empty(buf.fused_workspace_bytes(T, H, K, E, N1, mode), dtype=torch.uint8, device=dev)
    out = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    topk_w = torch.empty((T, K), dtype=torch.float32, device=dev)
    ids32 = torch.empty((T, K), dtype=torch.int32, device=dev)   # the router writes the type the fused operator takes
    nums = torch.empty(E, dtype=torch.int64, device=dev)

    ti = capi.tensor_info
    null = capi.TensorInfo()
    wdt = {1: None, 2: capi.DT_FP8_E4M3, 3: capi.DT_INT4X2}[mode]
    d = dict(x=ti(x), logits=ti(logits), w=ti(topk_w), ids=ti(ids32),
             w1=ti(w1, dtype=wdt, weight_format=capi.WEIGHT_FORMAT_PREPACKED), s1=ti(s1),
             w2=ti(w2, dtype=wdt, weight_format=capi.WEIGHT_FORMAT_PREPACKED), s2=ti(s2),
             out=ti(out), nums=ti(nums), ws=ti(ws))
    r = ctypes.byref
    st = capi.stream_ptr()

    def step():
        capi.check("route", lib.zbal_moe_topk_route(r(d["logits"]), K, r(d["ids"]), r(d["w"]), buf.comm, st, 0))
        capi.check("fused", lib.zbal_fused_deep_moe(
            r(d["x"]), r(d["ids"]), r(d["w1"]), r(d["s1"]), r(d["w2"]), r(d["s2"]), r(d["w"]), r(null), r(null), r(null),
            r(null), r(null), r(null), r(null), r(d["out"]), r(null), r(d["nums"]), r(d["ws"]), E, mode, 0, N1, 0, 0,
            buf.comm, st, 0))

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(args.steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    ms_per_step = e0.elapsed_time(e1) / args.steps
    out_fused = out.clone()

    # ---- the same stages one by one through the inner kernel ABI, with events between them -----------------
    off = {k: int(v) for k, v in plan_workspace(lib, T, H, K, E, N1, mode).items()}
    base = ws.data_ptr()
    q1, xs, eidx, row_off, q2, sc2, y = (base + off[k] for k in ("q1", "xs", "expand_idx", "row_off", "q2", "scale2", "y"))
    lscratch = base + off["layout_scratch"]
    sgl = base + off["sgl"] if mode != 2 else None
    rowmax = sgl + rows * I * 4 if sgl else None      # int modes: row maxima behind the fp32 SwiGLU values; the permute launch clears them
    names = ["route", "permute_quant", "gmm1_swiglu_quant", "gmm2_dequant", "combine"]
    s2dt = {1: capi.DT_BF16, 2: capi.DT_FP32, 3: capi.DT_FP16}[mode]

    y_window = (ctypes.c_void_p * 1)(y)        # the one rank's window the expert outputs sit in

    def staged(evs):
        evs[0].record()
        capi.check("route", lib.zbalhip_topk_route(logits.data_ptr(), T, E, K, ids32.data_ptr(), 0, topk_w.data_ptr(), st))
        evs[1].record()
        capi.check("permute", lib.zbalhip_fused_permute_quant(x.data_ptr(), capi.DT_BF16, ids32.data_ptr(), None, None, T, H, K, E,
                                                              2 if mode == 2 else 1, q1, xs, eidx, nums.data_ptr(), row_off,
                                                              rowmax, rows if rowmax else 0, lscratch, 50, st))
        evs[2].record()
        capi.check("gmm1", lib.zbalhip_gmm1_swiglu_quant(q1, xs, w1.data_ptr(), s1.data_ptr(), row_off, E, rows, H, N1,
                                                         mode | (capi.ROWMAX_CLEARED if rowmax else 0),
                                                         q2, sc2, sgl, st))
        evs[3].record()
        capi.check("gmm2", lib.zbalhip_gmm2_dequant(q2, sc2, w2.data_ptr(), s2.data_ptr(), s2dt, row_off, E, rows, I,
                                                    H, mode, capi.DT_BF16, y, st))
        evs[4].record()
        capi.check("combine", lib.zbalhip_combine(y_window, 1, 0, rows, capi.DT_BF16, row_off, 0, topk_w.data_ptr(),
                                                  ids32.data_ptr(), eidx, T, H, K, E, out.data_ptr(), st))
        evs[5].record()

    all_evs = [[torch.cuda.Event(enable_timing=True) for _ in range(6)] for _ in range(args.steps)]
    for _ in range(max(1, args.warmup // 2)):
        staged([torch.cuda.Event(enable_timing=True) for _ in range(6)])
    torch.cuda.synchronize()
    for evs in all_evs:
        staged(evs)
    torch.cuda.synchronize()
    stage_ms = {n: sum(evs[i].elapsed_time(evs[i + 1]) for evs in all_evs) / args.steps for i, n in enumerate(names)}
    assert torch.equal(out, out_fused), "staged and fused paths disagree"

    flops1 = 2.0 * rows * H * N1
    flops2 = 2.0 * rows * I * H
    qbytes = rows * (H + (H // 128 * 4 if mode == 2 else 4))
    bytes_permute = T * H * 2 + qbytes
    bytes_combine = rows * H * 2 + T * H * 2
    t1 = stage_ms["gmm1_swiglu_quant"] * 1e-3
    t2 = stage_ms["gmm2_dequant"] * 1e-3
    if workload == "decode":
        # a handful of rows per expert: the GEMMs stream the weights of the experts that received tokens
        touched = int((nums > 0).sum().item())
        wbytes1 = touched * H * N1
        roofline = {"kernel": "grouped_gemm_dma_kernel<int8, gmm1>", "bound": "hbm", "achieved": wbytes1 / t1 / 1e9,
                    "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": wbytes1 / t1 / 1e9 / PEAK_HBM_GBS, "traffic": None,
                    "experts_with_tokens": touched}
    else:
        kname = "grouped_gemm_dma_kernel<%s, gmm1>" % {1: "int8", 2: "fp8", 3: "w4a8"}[mode]
        routed = workload in ("prefill", "qwen_w4a8") and T == cfg["T"] and not args.equal_rows
        roofline = {"kernel": kname, "bound": "mfma", "achieved": flops1 / t1 / 1e12,
                    "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s" if mode == 2 else "TOP/s",
                    "frac": flops1 / t1 / 1e12 / PEAK_FP8_TFLOPS,
                    "traffic": measured_traffic(workload + "_gmm1") if routed else None}
    stages = {
        "ms": {k: round(v, 4) for k, v in stage_ms.items()},
        "gmm1_tflops": flops1 / t1 / 1e12,
        "gmm2_tflops": flops2 / t2 / 1e12,
        "permute_quant_gbs": bytes_permute / (stage_ms["permute_quant"] * 1e-3) / 1e9,
        "combine_gbs": bytes_combine / (stage_ms["combine"] * 1e-3) / 1e9,
        "permute_quant_frac_hbm": bytes_permute / (stage_ms["permute_quant"] * 1e-3) / 1e9 / PEAK_HBM_GBS,
        "combine_frac_hbm": bytes_combine / (stage_ms["combine"] * 1e-3) / 1e9 / PEAK_HBM_GBS,
    }

    # ---- CPU baseline on a bounded sample, which also checks the GPU result -------------------------------------
    cpu = None
    parity = None
    if not args.no_cpu:
        from oracle import oracle as zo
        ts = min(args.cpu_sample_tokens if workload == "prefill" else 128, T)

        def h16(t):
            return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
        xs_np, ids_np, w_np = h16(x[:ts]), ids32[:ts].cpu().numpy(), topk_w[:ts].cpu().numpy()
        if mode == 2:
            w1_np, w2_np = w1_logical.view(torch.uint8).cpu().numpy(), w2_logical.view(torch.uint8).cpu().numpy()
            s1_np, s2_np = s1.cpu().numpy(), s2.cpu().numpy()
        else:
            w1_np, w2_np = w1_logical.cpu().numpy(), w2_logical.cpu().numpy()
            s1_np = s1.cpu().numpy() if mode == 1 else h16(s1)
            s2_np = h16(s2)
        t0 = time.perf_counter()
        ref, _ = zo.fused_moe(xs_np, zo.DT_BF16, ids_np, w_np, w1_np, s1_np, w2_np, s2_np, E, mode)
        secs = time.perf_counter() - t0
        got_bits = h16(out_fused[:ts])
        got, want = zo.bf16_to_f32(got_bits), zo.bf16_to_f32(ref)
        err = float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))
        big = np.abs(want) >= np.abs(want).max() / 64.0       # element-wise figure over the elements of appreciable size
        elem = float((np.abs(got - want)[big] / np.abs(want)[big]).max())
        parity = {"tokens": ts, "max_rel_err": err, "max_elem_rel_err_above_1_64_of_max": elem, "tolerance": 2e-2,
                  "ok": bool(err < 2e-2),
                  "bit_exact": bool(np.array_equal(got_bits, ref))}
        cpu = {"value": ts / secs, "unit": "tokens/s", "cores": zo.num_threads(), "kind": "port",
               "sample": "first %d tokens of the same batch (%d expert rows, all %d experts' weights), %.1f s" %
                         (ts, ts * K, E, secs)}

    line = {
        "metric": "MoE layer tokens/s at 1 GPU", "value": T / (ms_per_step * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": cfg["dtype"], "data": "synthetic",
        "config": {"workload": cfg["name"], "tokens": T, "hidden": H, "experts": E, "topk": K, "intermediate": I,
                   "quant": cfg["quant"], "parallelism": "1 GPU", "l2_flush_between_steps": False,
                   "routing": "equal rows per expert (profiling)" if (workload == "prefill" and args.equal_rows) else
                              ("uniform-random logits" if cfg["zipf"] is None else "Zipf(%.1f) popularity" % cfg["zipf"])},
        "roofline": roofline, "cpu_baseline": cpu, "stages": stages, "parity": parity,
    }
    return line


def bench_reduce(args, torch, np, capi, buf):
    """BASELINE configs[3]: one rank's reduce-scatter shard, 8 peer buffers of 256 MiB held as local HBM
    allocations, through zbal_reduce_scatter. Algorithmic bytes = (8 + 1) x 256 MiB = 2.416 GB per launch."""
    from memfabric_hybrid_amd.operators import create_group, destroy_group
    lib = buf.lib
    R, nbytes = 8, 256 << 20
    comm = create_group("bench_rs8", R, 0)
    st = capi.stream_ptr()
    results = {}
    for name, tdt, zdt in (("bf16", torch.bfloat16, capi.DT_BF16), ("fp32", torch.float32, capi.DT_FP32)):
        n = nbytes // torch.empty(0, dtype=tdt).element_size()
        peers = [torch.randn(n, device="cuda", dtype=torch.float32).to(tdt) if tdt != torch.float32
                 else torch.randn(n, device="cuda", dtype=tdt) for _ in range(R)]
        out = torch.empty(n, device="cuda", dtype=tdt)
        for r in range(R):
            capi.check("window", lib.zbal_comm_register_peer_window(comm, r, peers[r].data_ptr(), nbytes))

        def step():
            capi.check("reduce_scatter", lib.zbal_reduce_scatter(peers[0].data_ptr(), out.data_ptr(), n, zdt,
                                                                 capi.REDUCE_SUM, comm, st))
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            step()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / args.steps
        # fixed-order fp32 accumulation, one rounding: torch's sequential sum in fp32 is the same arithmetic
        ref = peers[0].float()
        for r in range(1, R):
            ref = ref + peers[r].float()
        ok = bool(torch.equal(ref.to(tdt), out))
        results[name] = {"ms": ms, "gbs": (R + 1) * nbytes / (ms * 1e-3) / 1e9, "exact": ok}
        # a one-input "reduction" is a plain copy of known traffic (2 x 256 MiB): the calibration point for
        # the FETCH_SIZE / WRITE_SIZE counters
        arr = (ctypes.c_void_p * 1)(peers[1].data_ptr())
        capi.check("copy", lib.zbalhip_reduce(arr, 1, n, zdt, capi.REDUCE_SUM, out.data_ptr(), 0, None, 0, st))
        torch.cuda.synchronize()
        del peers, out, ref
    destroy_group(comm)
    b = results["bf16"]
    line = {"metric": "local N-buffer reduce GB/s at 1 GPU", "value": b["gbs"], "unit": "GB/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": b["ms"], "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "bf16 in, fp32 accumulate, bf16 out", "data": "synthetic",
            "config": {"workload": "local reduce-scatter shard (BASELINE configs[3])", "buffers": R,
                       "bytes_per_buffer": nbytes},
            "roofline": {"kernel": "reduce_kernel<bf16, sum, 8>", "bound": "hbm", "achieved": b["gbs"], "peak": PEAK_HBM_GBS,
                         "unit": "GB/s", "frac": b["gbs"] / PEAK_HBM_GBS, "traffic": measured_traffic("reduce_8x256MiB_bf16")},
            "cpu_baseline": None, "variants": results}
    return line


def plan_workspace(lib, T, H, K, E, N1, qmode):
    """Offsets of the fused operator's workspace regions; mirrors PlanFusedWorkspace in the host layer
    (csrc/host/zbal_gpu_communicator.cpp) and is cross-checked against the size the library reports."""
    rows = max(T * K, 1)
    I = N1 // 2
    fp8 = qmode == 2
    off = {}
    cur = 0

    def take(name, nbytes):
        nonlocal cur
        off[name] = cur
        cur = (cur + nbytes + 255) & ~255

    take("q1", rows * H)
    take("xs", rows * (H // 128 if fp8 else 1) * 4)
    take("expand_idx", rows * 4)
    take("counts", E * 8)
    take("row_off", (E + 1) * 4)
    take("layout_scratch", 50 * E * 4)
    take("q2", rows * I)
    take("scale2", rows * ((I + 127) // 128 if fp8 else 1) * 4)
    if not fp8:
        take("sgl", rows * (I + 1) * 4)
    take("y", rows * H * 2)
    assert cur == lib.zbal_fused_deep_moe_workspace_size(T, H, K, E, N1, 0, qmode), "workspace plan out of sync"
    return off


if __name__ == "__main__":
    main()
