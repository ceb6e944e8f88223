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

# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this same command
# (profiles/momoe_layer_headline_{fetch,write}_size.txt; fetch scaled x2.0, write x1.0 by the
# 256 MiB copy in the same runs).  Counters cannot be read from inside this process, so these are
# the figures of the profile run named in TRAFFIC_SOURCE, not of the run that prints them; None
# for a kernel that has not been measured.
TRAFFIC_SOURCE = "profiles/momoe_layer_headline_fetch_size.txt + _write_size.txt"
MEASURED_TRAFFIC_BYTES = {
    "momoe_lin1_swiglu_fwd": 2 * 708812 * 1024 + 148256 * 1024,
    "momoe_lin2_scale_fwd": 2 * 425536 * 1024 + 271259 * 1024,
    "momoe_dgrad_h": 2 * 388726 * 1024 + 131943 * 1024,
    "momoe_lin1_swiglu_bwd": 2 * 915365 * 1024 + 402186 * 1024,
    "momoe_wgrad[Wl2]": 2 * 238101 * 1024 + 524315 * 1024,
    "momoe_wgrad[Wl1]": 2 * 295637 * 1024 + 1048598 * 1024,
    "momoe_dgrad_x": 2 * 710413 * 1024 + 262144 * 1024,
}


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


def cpu_baseline(D, H, N, K, budget_s=25.0):
    """The oracle MoE layer as `MoE.forward` runs it (router -> per-expert loop -> bias update,
    momoe/sample_moe.py:59-68) plus its autograd backward, in fp32 on the host cores, on a
    reduced token count of the same layer."""
    import torch
    import oracle
    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    Ms = 1024
    x, W1, W2, _, _, dy = headline_inputs(Ms, D, H, N, K, seed=1)
    Wg = torch.randn(D, N, generator=torch.Generator().manual_seed(2)) / D ** 0.5
    moe = oracle.OracleMoE(D, H, N, K, 0, Wg_DN=Wg, Wl1_ND2H=W1.float(), Wl2_NHD=W2.float())
    xf = x.bfloat16().float().reshape(1, Ms, D).requires_grad_()
    dyf = dy.reshape(1, Ms, D)
    times = []
    t_start = time.time()
    for it in range(4):
        t0 = time.time()
        y = moe(xf)
        y.backward(dyf)
        dt = time.time() - t0
        moe.zero_grad(set_to_none=True)
        xf.grad = None
        if it > 0:
            times.append(dt)
        if time.time() - t_start > budget_s and times:
            break
    best = min(times)
    return {"value": Ms / best, "unit": "tokens/s", "cores": threads, "kind": "port",
            "sample": f"oracle MoE (router + experts + bias update) fwd+bwd, fp32, {Ms} of 8192 tokens of the "
                      f"headline layer (D={D}, H={H}, N={N}, K={K}), best of {len(times)} runs, {best:.3f} s each"}


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

    layer = make_layer(args.save_percent)
    ms = timed(layer, step, args.steps, args.warmup)
    ms_fwd = timed(layer, fwd_only, args.steps, 2)
    torch.cuda.reset_peak_memory_stats()
    base_mem = torch.cuda.memory_allocated()
    step(layer)
    torch.cuda.synchronize()
    peak_extra_mib = (torch.cuda.max_memory_allocated() - base_mem) / 2**20

    # per-kernel launch durations (HIP events on the launch stream) and the shader clock the
    # grouped GEMMs ran at (in-kernel counters), over `steps` more steps of the same loop
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
    n_sus = max(args.steps, int(2000.0 / ms) + 1)
    with _hip.clock_trace() as ct:
        ms_sustained = timed(layer, step, n_sus, 0)
    clock_sustained = ct.mhz()

    # the same step captured once in a HIP graph and replayed (launch gaps only; the routing may
    # change between replays: no launch is sized from it on the host)
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
    roofline = {"bound": "mfma", "kernel": dom, "achieved": kernels[dom]["tflops"], "peak": PEAK_BF16_TFLOPS,
                "unit": "TFLOP/s", "frac": kernels[dom]["tflops"] / PEAK_BF16_TFLOPS,
                "avg_launch_ms": kernels[dom]["avg_ms"], "traffic": MEASURED_TRAFFIC_BYTES.get(dom),
                "traffic_source": TRAFFIC_SOURCE if dom in MEASURED_TRAFFIC_BYTES else None,
                "shader_clock_mhz": clock_timed}

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
        "roofline": roofline, "kernels": kernels,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(D, H, N, K)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
