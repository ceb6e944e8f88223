"""Benchmark of the MoE-layer hot path on one MI355X.

One step = one forward + backward of `MoMoE` (x, mask, s -> y; dy -> dx, dWl1, dWl2, ds)
on the headline layer: B=4, S=2048 (8192 tokens), D=2048, H=1024, N=128 experts, K=8,
bf16 with fp32 accumulation, save_percent=0.  Inputs are synthetic, seeded, and resident
in HBM before the timed region.  Prints ONE JSON line: the headline figure from exactly
`--steps` timed steps, and next to it the forward alone, the other save setting, a sustained
figure from at least 2 s of back-to-back steps, the shader clock the GEMMs ran at, the layer
with its router in front, per-kernel launch times with their fraction of the MFMA or HBM
roofline, and the CPU oracle on the host cores.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "momoe-impl_amd"), os.path.join(ROOT, "tests")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0

# HBM bytes per launch come from two rocprofv3 --pmc runs of this same command (FETCH_SIZE, then
# WRITE_SIZE, KiB per dispatch), whose summaries are kept as text under profiles/ together with
# the factor that the 256 MiB copy of --calibrate-copy gives each counter ("== scale:" line).
# Counters cannot be read from inside this process, so the figures are those of the profiled run,
# not of the run that prints them: they are parsed from the summaries every time, never typed in.
TRAFFIC_FILES = {"fetch": "profiles/momoe_layer_headline_fetch_size.txt",
                 "write": "profiles/momoe_layer_headline_write_size.txt"}
TRAFFIC_SOURCE = " + ".join(TRAFFIC_FILES.values())
# kernel names in the summaries -> entry points as this file names them
PROFILE_KERNELS = {
    "lin1_swiglu_kernel[fwd]": "momoe_lin1_swiglu_fwd", "lin1_swiglu_kernel[bwd]": "momoe_lin1_swiglu_bwd",
    "lin2_scale_kernel": "momoe_lin2_scale_fwd", "dgrad_h_kernel": "momoe_dgrad_h",
    "dgrad_x_kernel": "momoe_dgrad_x", "wgrad_kernel[Wl1": "momoe_wgrad[Wl1]",
    "wgrad_kernel[Wl2": "momoe_wgrad[Wl2]", "combine_kernel": "momoe_combine",
}


def parse_counter_summary(path, counter):
    """(scale, {kernel name in the summary: average counter value per dispatch})."""
    scale, rows = None, {}
    with open(path) as f:
        for line in f:
            if line.startswith("== scale:"):
                scale = float(line.split(":", 1)[1].split()[0])
            elif f" {counter} " in line and not line.startswith(("#", "==")):
                name, rest = line.split(f" {counter} ", 1)
                rows[name.strip()] = float(rest.split()[0])
    if scale is None:
        raise ValueError(f"{path}: no '== scale:' line")
    return scale, rows


def measured_traffic(root=ROOT):
    """{entry point: HBM bytes per launch = scale_f * FETCH_SIZE + scale_w * WRITE_SIZE} from the
    committed counter summaries; empty when they are not there."""
    try:
        sf, fetch = parse_counter_summary(os.path.join(root, TRAFFIC_FILES["fetch"]), "FETCH_SIZE")
        sw, write = parse_counter_summary(os.path.join(root, TRAFFIC_FILES["write"]), "WRITE_SIZE")
    except (OSError, ValueError):
        return {}
    out = {}
    for prof_name, entry in PROFILE_KERNELS.items():
        f = [v for k, v in fetch.items() if k.startswith(prof_name)]
        w = [v for k, v in write.items() if k.startswith(prof_name)]
        if len(f) == 1 and len(w) == 1:
            out[entry] = int(round((sf * f[0] + sw * w[0]) * 1024))
    return out


MEASURED_TRAFFIC_BYTES = measured_traffic()


def headline_inputs(M, D, H, N, K, seed=0):
    import torch
    from helpers import make_routing
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, D, generator=g)
    dy = torch.randn(M, D, generator=g)
    W1 = torch.empty(N, D, 2 * H, dtype=torch.bfloat16).normal_(0, 0.02, generator=g)
    W2 = torch.empty(N, H, D, dtype=torch.bfloat16).normal_(0, 0.02, generator=g)
    mask, s = make_routing(M, N, K, 0, seed=seed)
    return x, W1, W2, mask, s, dy


def kernel_flops(D, H, msum):
    """Algorithmic flops per launch (2*m*n*k per GEMM; recomputation counted separately)."""
    unit = float(D) * H * msum
    return {
        "momoe_lin1_swiglu_fwd": 4 * unit, "momoe_lin2_scale_fwd": 2 * unit,
        "momoe_dgrad_h": 2 * unit, "momoe_lin1_swiglu_bwd": 4 * unit, "momoe_dgrad_x": 4 * unit,
        "momoe_wgrad[Wl2]": 2 * unit, "momoe_wgrad[Wl1]": 4 * unit,
    }


def gemm_algorithmic_bytes(M, D, H, N, K):
    """Bytes a GEMM launch must move at least: every input read once, every output written once
    (weights 2 bytes per element; x and G_y are read once although gathered)."""
    msum = M * K
    w1, w2 = N * D * 2 * H * 2, N * H * D * 2
    xb, hb, ysb, gzb = M * D * 2, msum * H * 2, msum * D * 2, msum * 2 * H * 2
    return {
        "momoe_lin1_swiglu_fwd": w1 + xb + hb,
        "momoe_lin2_scale_fwd": w2 + hb + ysb,
        "momoe_dgrad_h": w2 + xb + hb,
        "momoe_lin1_swiglu_bwd": w1 + xb + hb + gzb + hb + msum * 4 * ((H + 127) // 128),
        "momoe_wgrad[Wl2]": hb + xb + w2,
        "momoe_wgrad[Wl1]": xb + gzb + w1,
        "momoe_dgrad_x": w1 + gzb + ysb,
    }


def kernel_bytes(M, D, H, N, K):
    """Algorithmic HBM bytes per launch of the bandwidth-bound kernels."""
    msum = M * K
    return {
        # mask once, idx + inv (the reference's idx + which), cumsums, sizes
        "momoe_index_build": N * M * 4 + 2 * msum * 4 + (N + 1) * 4 + N * 8,
        # prefix sums in, one 16-byte entry per 256-row tile out (launch-bound: a few microseconds)
        "momoe_tile_table_build": (N + 1) * 4 + 16 * (msum // 256 + N),
        "momoe_combine": msum * D * 2 + M * D * 2 + msum * 4,
        "momoe_gs_scatter": msum * ((H + 127) // 128) * 4 + msum * 4 + msum * 4,
        # bf16 logits in; mask, s, p_sel out (4 bytes each); Ng, Ks per token
        "momoe_router_fwd": M * N * (2 + 12) + M * 8 + N * 4,
        # G_s, p_sel, s, mask in (4 bytes each); bf16 logit gradient out
        "momoe_router_bwd": M * N * (16 + 2) + M * 8,
        # saved a|b and u in; gz, hs out; one partial sum per row
        "momoe_swiglu_bwd_saved": msum * H * 2 * (2 + 1 + 2 + 1) + msum * 4,
    }


def _host_cpus():
    """(logical CPUs the OS shows, physical cores, CPUs this process may run on)."""
    logical = os.cpu_count() or 1
    try:
        import psutil
        physical = psutil.cpu_count(logical=False) or logical
    except Exception:
        physical = logical
    try:
        usable = len(os.sched_getaffinity(0))
    except Exception:
        usable = logical
    return logical, physical, usable


def _oracle_moe_pass(oracle, torch, x, Wg, W1, W2, biases, dy, K, dtype, backward):
    """One pass of the oracle MoE layer as `MoE.forward` runs it (router -> experts -> bias
    update, momoe/sample_moe.py:59-68) and, with `backward`, its backward (experts, then router:
    momoe/momoe.py:881-903, momoe/topk_router.py:127-145), every product formed once."""
    M, D = x.shape
    N = W1.shape[0]
    r = oracle.router_forward(x, Wg, biases, N, K, 0)
    mask, s = r["mask_NM"], r["s_NM"]
    if not backward:
        y = oracle.experts_forward(x, W1, W2, mask, s, dtype=dtype)
        oracle.bias_update(biases, (mask != 0).sum(1), M, K, 0, 1e-4)
        return y
    y, G_x, G_W1, G_W2, G_s = oracle.experts_forward_backward(x, W1, W2, mask, s, dy, dtype=dtype)
    oracle.bias_update(biases, (mask != 0).sum(1), M, K, 0, 1e-4)
    G_logit = oracle.router_backward_closed_form(G_s.float(), r["p_sel_MN"], s, r["Ng_M"], r["Ks_M"],
                                                 mask, 0, round_bf16=True).to(dtype)
    Wgd, xd = Wg.to(dtype), x.to(dtype)
    G_x = G_x + G_logit @ Wgd.T
    G_Wg = xd.T @ G_logit
    return y, G_x, G_W1, G_W2, G_Wg


def cpu_baseline(D, H, N, K, budget_s=28.0):
    """The CPU restatement of `MoE.forward` (router -> per-expert loop -> bias update) and of its
    backward, timed on the host cores: forward and forward+backward, fp32 and bf16, on the tiny
    reference configuration and on a 1024-token slice of the headline layer.  `value` is the
    fp32 forward+backward rate of the headline slice.  A plain torch.mm on the same threads is
    timed beside it, so the figure can be read against what these cores give a GEMM."""
    import torch
    import oracle
    from helpers import make_layer_inputs
    logical, physical, usable = _host_cpus()
    # the threads torch starts with: OMP_NUM_THREADS where the machine sets it (a box shared
    # between jobs says there how many cores are this job's), else every CPU of the process
    threads = torch.get_num_threads()
    t_begin = time.time()

    def best_of(fn, cap_s, min_runs=3, max_runs=5):
        fn()  # warm-up (page faults, thread pool start)
        times = []
        t0 = time.time()
        while len(times) < max_runs and (len(times) < min_runs or time.time() - t0 < cap_s):
            t = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t)
            if time.time() - t0 > 2.5 * cap_s:
                break
        return min(times), len(times)

    def mm_rate(m, k, n, dtype):
        a, b = torch.randn(m, k).to(dtype), torch.randn(k, n).to(dtype)
        t, _ = best_of(lambda: torch.mm(a, b), 0.5, 3, 10)
        return 2.0 * m * k * n / t / 1e9

    results = {}
    # C1: the reference's own CPU-sized case (B=2, S=64, D=128, H=64, N=8, K=2)
    tiny = dict(M=128, D=128, H=64, N=8, K=2)
    # the headline layer at 1024 of its 8192 tokens: every expert, 64 rows per expert on average
    slice_ = dict(M=1024, D=D, H=H, N=N, K=K)
    for label, c in (("tiny", tiny), ("headline_slice", slice_)):
        x, W1, W2, _, _, dy = make_layer_inputs(c["M"], c["D"], c["H"], c["N"], c["K"], seed=1)
        x = x.bfloat16().float()
        Wg = (torch.randn(c["D"], c["N"], generator=torch.Generator().manual_seed(2)) / c["D"] ** 0.5).bfloat16()
        biases = torch.zeros(c["N"])
        unit = float(c["D"]) * c["H"] * c["M"] * c["K"]
        for dtype, dname in ((torch.float32, "fp32"), (torch.bfloat16, "bf16")):
            W1d, W2d, xd, dyd = W1.to(dtype), W2.to(dtype), x.to(dtype), dy.to(dtype)
            for backward in (False, True):
                left = budget_s - (time.time() - t_begin)
                cap = 0.2 if label == "tiny" else max(0.5, left / (5 if dtype == torch.float32 else 3))
                with torch.no_grad():
                    t, n = best_of(lambda: _oracle_moe_pass(oracle, torch, xd, Wg, W1d, W2d, biases, dyd,
                                                            c["K"], dtype, backward), cap)
                key = f"{label}_{dname}_{'fwd_bwd' if backward else 'fwd'}"
                results[key] = {"tokens_per_s": c["M"] / t, "seconds": t, "runs": n,
                                "gflops": (18.0 if backward else 6.0) * unit / t / 1e9}
            del W1d, W2d
    rows = slice_["M"] * K // N

    def mm_rate_streaming(dtype):
        # the up projection of the slice as the layer meets it: one [rows, D] x [D, 2H] product
        # per expert, each with its own weights (N * D * 2H elements streamed from memory)
        a, w = torch.randn(rows, D).to(dtype), W1.to(dtype)
        t, _ = best_of(lambda: [torch.mm(a, w[i]) for i in range(N)], 0.5, 3, 5)
        return 2.0 * rows * D * 2 * H * N / t / 1e9

    results["torch_mm_gflops"] = {
        f"fp32_[{rows},{D}]x[{D},{2 * H}]_one_weight_in_cache": mm_rate(rows, D, 2 * H, torch.float32),
        f"fp32_[{rows},{D}]x[{D},{2 * H}]_per_expert_weights": mm_rate_streaming(torch.float32),
        "fp32_[2048,2048]x[2048,2048]": mm_rate(2048, 2048, 2048, torch.float32),
        f"bf16_[{rows},{D}]x[{D},{2 * H}]_per_expert_weights": mm_rate_streaming(torch.bfloat16),
    }
    head = results["headline_slice_fp32_fwd_bwd"]
    return {"value": head["tokens_per_s"], "unit": "tokens/s", "cores": threads, "kind": "port",
            "logical_cpus": logical, "physical_cores": physical, "usable_cpus": usable,
            "torch_threads": threads,
            "sample": f"CPU oracle of the MoE layer (router + experts + bias update; backward: experts then "
                      f"router), every GEMM executed once (18*D*H flops per pair, no autograd), on "
                      f"{threads} torch threads ({physical} physical / {logical} logical CPUs on the host, "
                      f"{usable} usable by this process): value = fp32 forward+backward of {slice_['M']} of "
                      f"the 8192 tokens of the headline layer (D={D}, H={H}, N={N}, K={K}; {rows} rows per "
                      f"expert), best of {head['runs']} runs of {head['seconds']:.3f} s = "
                      f"{head['gflops']:.0f} GFLOP/s; `variants` holds fp32 and bf16, forward and "
                      f"forward+backward, for that slice and for the tiny reference configuration "
                      f"(128 tokens, D=128, H=64, N=8, K=2), and torch.mm rates on the same threads",
            "variants": results}


def _mark(what):
    """Name the section that is about to use the GPU, on stderr and flushed: if a run dies there,
    the end of its output says where."""
    print(f"[bench] {what}", file=sys.stderr, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--save-percent", type=float, default=0)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a 256 MiB device-to-device copy a few times, so that a "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE run of this command contains a "
                         "kernel of known traffic to scale the counters by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU only: this build has no multi-GPU path "
              "(run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    import momoe_amd
    from momoe_amd import _hip

    B, S, D, H, N, K = 4, 2048, 2048, 1024, 128, 8
    M = B * S
    msum = M * K
    dev = "cuda:0"
    x, W1, W2, mask, s, dy = headline_inputs(M, D, H, N, K)
    maskd = mask.to(dev)
    sd = s.T.contiguous().to(dev).T.requires_grad_()
    xd = x.to(dev, torch.bfloat16).reshape(B, S, D).requires_grad_()
    dyd = dy.to(dev, torch.bfloat16).reshape(B, S, D)

    if args.calibrate_copy:
        src = torch.empty(128 * 2**20, dtype=torch.bfloat16, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    def make_layer(sp):
        return momoe_amd.MoMoE(D, H, N, K, save_percent=sp, Wl1_ND2H=W1.to(dev), Wl2_NHD=W2.to(dev))

    def step(layer):
        y, _ = layer(xd, maskd, sd)
        y.backward(dyd)
        layer.Wl1_ND2H.grad = layer.Wl2_NHD.grad = xd.grad = sd.grad = None

    def timed(layer, fn, steps, warmup):
        for _ in range(warmup):
            fn(layer)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn(layer)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps

    def fwd_only(layer):
        with torch.no_grad():
            layer(xd, maskd, sd)

    _mark("headline step, timed")
    layer = make_layer(args.save_percent)
    ms = timed(layer, step, args.steps, args.warmup)
    _mark("forward only")
    ms_fwd = timed(layer, fwd_only, args.steps, 2)
    torch.cuda.reset_peak_memory_stats()
    base_mem = torch.cuda.memory_allocated()
    step(layer)
    torch.cuda.synchronize()
    peak_extra_mib = (torch.cuda.max_memory_allocated() - base_mem) / 2**20

    # per-kernel launch durations (HIP events on the launch stream) and the shader clock the
    # grouped GEMMs ran at (in-kernel counters), over `steps` more steps of the same loop
    _mark("per-kernel launch times and shader clock")
    per = {}
    with _hip.clock_trace() as ct, _hip.kernel_timer() as kt:
        for _ in range(args.steps):
            step(layer)
    clock_timed = ct.mhz()

    def collect(kt, per):
        wcount = 0
        for name, t in kt.durations_ms():
            if name == "momoe_wgrad":
                name = "momoe_wgrad[Wl2]" if wcount % 2 == 0 else "momoe_wgrad[Wl1]"
                wcount += 1
            per.setdefault(name, []).append(t)

    collect(kt, per)

    # sustained rate: at least 2 s of back-to-back steps (the timed region above is a burst of
    # a few tens of milliseconds, and these kernels run against the power limit)
    _mark("sustained steps")
    n_sus = max(args.steps, int(2000.0 / ms) + 1)
    with _hip.clock_trace() as ct:
        ms_sustained = timed(layer, step, n_sus, 0)
    clock_sustained = ct.mhz()

    # the same step captured once in a HIP graph and replayed (launch gaps only; the routing may
    # change between replays: no launch is sized from it on the host)
    _mark("graph capture and replay")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(layer)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(layer)
    ms_graph = timed(layer, lambda _l: graph.replay(), args.steps, args.warmup)
    del graph

    # the other save setting
    _mark("other save_percent")
    other_sp = 100 if args.save_percent == 0 else 0
    layer2 = make_layer(other_sp)
    ms_other = timed(layer2, step, max(args.steps // 2, 3), 2)
    if other_sp == 100:
        with _hip.kernel_timer() as kt2:
            for _ in range(3):
                step(layer2)
        for name, t in kt2.durations_ms():
            if name == "momoe_swiglu_bwd_saved":
                per.setdefault(name, []).append(t)
    del layer2

    # the layer with its router in front: MoE = TopKRouter -> MoMoE -> bias update
    # (momoe/sample_moe.py:59-68), gate weights ~ N(0, 1/D)
    _mark("layer with its router")
    Wg = torch.randn(D, N, generator=torch.Generator().manual_seed(3)) / D ** 0.5
    moe = momoe_amd.MoE(D, H, N, K, 0, save_percent=args.save_percent, Wg_DN=Wg.to(dev),
                        Wl1_ND2H=layer.Wl1_ND2H.data, Wl2_NHD=layer.Wl2_NHD.data)

    def moe_step(m):
        y = m(xd)
        y.backward(dyd)
        m.zero_grad(set_to_none=True)
        xd.grad = None

    ms_moe = timed(moe, moe_step, args.steps, 3)
    with _hip.kernel_timer() as kt3:
        for _ in range(args.steps):
            moe_step(moe)
    for name, t in kt3.durations_ms():
        if name.startswith("momoe_router"):
            per.setdefault(name, []).append(t)
    del moe

    launches = {k: len(v) / args.steps for k, v in per.items()}
    launches["momoe_swiglu_bwd_saved"] = 1.0
    kernels = {k: {"launches_per_step": launches[k], "avg_ms": sum(v) / len(v)} for k, v in per.items()}
    flops = kernel_flops(D, H, msum)
    for k, f in flops.items():
        if k in kernels:
            kernels[k]["tflops"] = f / kernels[k]["avg_ms"] / 1e9
            kernels[k]["frac_peak"] = kernels[k]["tflops"] / PEAK_BF16_TFLOPS
    for k, b in kernel_bytes(M, D, H, N, K).items():
        if k in kernels:
            kernels[k]["algorithmic_bytes"] = b
            kernels[k]["hbm_gbs"] = b / kernels[k]["avg_ms"] / 1e6
            kernels[k]["frac_hbm_peak"] = kernels[k]["hbm_gbs"] / PEAK_HBM_GBS
    dom = max((k for k in kernels if k in flops),
              key=lambda k: kernels[k]["avg_ms"] * kernels[k]["launches_per_step"])
    alg_bytes = gemm_algorithmic_bytes(M, D, H, N, K)
    for k, b in alg_bytes.items():
        if k in kernels:
            kernels[k]["algorithmic_bytes"] = b
            if k in MEASURED_TRAFFIC_BYTES:
                kernels[k]["traffic_bytes"] = MEASURED_TRAFFIC_BYTES[k]
                kernels[k]["traffic_over_algorithmic"] = MEASURED_TRAFFIC_BYTES[k] / b
    roofline = {"bound": "mfma", "kernel": dom, "achieved": kernels[dom]["tflops"], "peak": PEAK_BF16_TFLOPS,
                "unit": "TFLOP/s", "frac": kernels[dom]["tflops"] / PEAK_BF16_TFLOPS,
                "avg_launch_ms": kernels[dom]["avg_ms"], "traffic": MEASURED_TRAFFIC_BYTES.get(dom),
                "traffic_over_algorithmic": (MEASURED_TRAFFIC_BYTES[dom] / alg_bytes[dom]
                                             if dom in MEASURED_TRAFFIC_BYTES else None),
                "traffic_source": TRAFFIC_SOURCE if dom in MEASURED_TRAFFIC_BYTES else None,
                "shader_clock_mhz": clock_timed}

    # What this machine gives outside the timed region: the vendor library on the two forward
    # GEMMs at perfectly balanced experts (torch.bmm over N experts of Msum/N rows: no gather, no
    # epilogue, no ragged tiles), the weight stream alone, and the matrix pipe alone on register
    # operands of the layer's kind of data.  (Only products with untransposed operands: the
    # batched product with a transposed weight operand of the dL/dx shape ends in an illegal
    # memory access inside the vendor library on this software stack.)
    def event_ms(fn, n=10):
        for _ in range(3):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n

    R = msum // N
    gen = torch.Generator(device=dev).manual_seed(7)
    xa = torch.randn(N, R, D, generator=gen, device=dev).to(torch.bfloat16)
    ha = torch.randn(N, R, H, generator=gen, device=dev).to(torch.bfloat16)
    Wa, Wb = layer.Wl1_ND2H.data, layer.Wl2_NHD.data
    vendor = {"momoe_lin1_swiglu_fwd": lambda: torch.bmm(xa, Wa), "momoe_lin2_scale_fwd": lambda: torch.bmm(ha, Wb)}
    machine = {"vendor_gemm": f"torch.bmm over {N} experts of {R} rows each, bf16, N(0,1) activations: x.Wl1 and h.Wl2, "
                              "ms and TFLOP/s, and this library's launch on the real routing relative to it",
               "vendor_gemm_ms": {}, "vendor_gemm_tflops": {}, "this_library_over_vendor": {}}
    for k, fn in vendor.items():
        _mark(f"vendor GEMM for {k}")
        t = event_ms(fn)
        machine["vendor_gemm_ms"][k] = t
        machine["vendor_gemm_tflops"][k] = flops[k] / t / 1e9
        machine["this_library_over_vendor"][k] = kernels[k]["avg_ms"] / t
    del xa, ha, vendor
    _mark("weight stream probe")
    machine["hbm_read_stream_gbs"] = _hip.hbm_stream_probe(Wa)
    machine["hbm_read_stream"] = (f"the grouped GEMMs' weight stream alone (global -> LDS, four 16 KiB stages per CU "
                                  f"in flight) over Wl1, {Wa.numel() * 2 / 2**20:.0f} MiB")
    _mark("MFMA rate probe")
    for kind in ("gaussian", "zeros"):
        tf, mhz = _hip.mfma_rate_probe(kind)
        machine[f"mfma_only_tflops_{kind}"] = tf
        machine[f"mfma_only_shader_clock_mhz_{kind}"] = mhz

    useful = 18.0 * D * H * msum
    out = {
        "metric": "moe_layer_fwd_bwd_tokens_per_s", "value": M / (ms * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "headline MoE layer fwd+bwd: B=4 S=2048 (8192 tokens) D=2048 H=1024 "
                               "N=128 K=8, near-uniform top-8 routing of N(0,1) logits",
                   "save_percent": args.save_percent, "tokens": M, "D": D, "H": H, "experts": N, "top_k": K},
        "fwd_bwd_tflops": useful / ms / 1e9, "fwd_bwd_frac_bf16_peak": useful / ms / 1e9 / PEAK_BF16_TFLOPS,
        "fwd_ms": ms_fwd, "fwd_tokens_per_s": M / (ms_fwd * 1e-3),
        "fwd_tflops": 6.0 * D * H * msum / ms_fwd / 1e9,
        f"ms_per_step_save_percent_{other_sp}": ms_other,
        "graph_replay_ms_per_step": ms_graph,
        "sustained_ms_per_step": ms_sustained, "sustained_steps": n_sus,
        "sustained_tokens_per_s": M / (ms_sustained * 1e-3),
        "shader_clock_mhz": clock_timed, "sustained_shader_clock_mhz": clock_sustained,
        "ms_per_step_with_router": ms_moe, "tokens_per_s_with_router": M / (ms_moe * 1e-3),
        "peak_activation_mib": peak_extra_mib,
        "roofline": roofline, "machine": machine, "kernels": kernels,
    }
    if not args.no_cpu_baseline:
        _mark("CPU baseline (no GPU work)")
        out["cpu_baseline"] = cpu_baseline(D, H, N, K)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
