"""Timings of the other layer shapes of the benchmark plan on one MI355X: the Qwen3-shaped
inference forward at several token counts, the skewed routing with shared experts, and the
4096 x 2048 layer at save_percent 0 / 50 / 100.  (bench.py at the repository root measures
the headline shape and prints the one JSON line the driver reads; this script prints a table.)

Usage: python momoe-impl_amd/bench_configs.py            # the shapes above
       python momoe-impl_amd/bench_configs.py --only skewed   # one of: inference headline skewed large
       python momoe-impl_amd/bench_configs.py --vendor   # the vendor GEMM library on the forward GEMMs of the
                                                         # headline step at perfectly balanced experts, and the
                                                         # rate at which library kernels read HBM
       python momoe-impl_amd/bench_configs.py --chart    # the grid of the reference's README charts
                                                         # (momoe/images/moe_full.png, moe_forward.png,
                                                         # moe_memory.png): TF/s forward and
                                                         # forward+backward at save_percent 0/50/100 and
                                                         # the memory held between forward and backward
"""
import math
import os
import sys
import time

import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import momoe_amd  # noqa: E402
from momoe_amd import _hip  # noqa: E402

DEV = "cuda:0"


def routing(M, N, K, Ks, skew, gen):
    """mask_NM int32 [N,M], s_NM fp32 (transposed view): top-(K-Ks) of softmax(logits) over the
    routed experts, renormalised; the last Ks experts hold every token."""
    Ng = N - Ks
    logits = torch.randn(M, N, generator=gen, device=DEV)
    if skew:
        logits[:, :Ng] -= skew * torch.log(torch.arange(1, Ng + 1, device=DEV, dtype=torch.float32))
    p = torch.softmax(logits[:, :Ng], -1)
    sel = torch.topk(p, K - Ks, dim=-1).indices
    chosen = torch.zeros(M, Ng, dtype=torch.bool, device=DEV).scatter_(1, sel, True)
    w = p * chosen
    s_MN = torch.cat([w / w.sum(-1, keepdim=True), torch.softmax(logits[:, Ng:], -1)], -1)
    mask = torch.ones(N, M, dtype=torch.int32, device=DEV)
    mask[:Ng] = chosen.T.to(torch.int32)
    return mask.contiguous(), s_MN.contiguous().T


def balanced_routing(M, N, K, gen):
    """The M*K pairs dealt to the experts round-robin: pair j of token m goes to expert
    (m*K + j) mod N, K consecutive (hence distinct) experts per token, and every expert gets
    floor(M*K/N) or ceil(M*K/N) tokens whether or not K divides N."""
    assert K <= N
    cols = (torch.arange(M, device=DEV)[:, None] * K + torch.arange(K, device=DEV)[None, :]) % N
    chosen = torch.zeros(M, N, dtype=torch.bool, device=DEV).scatter_(1, cols, True)
    w = torch.rand(M, N, generator=gen, device=DEV) * chosen
    return chosen.T.to(torch.int32).contiguous(), (w / w.sum(-1, keepdim=True)).contiguous().T


def run(name, M, D, H, N, K, Ks=0, skew=None, sp=0, backward=True, steps=5, graph=False):
    gen = torch.Generator(device=DEV).manual_seed(1)
    x = torch.randn(M, D, generator=gen, device=DEV).to(torch.bfloat16).reshape(1, M, D)
    dy = torch.randn(M, D, generator=gen, device=DEV).to(torch.bfloat16).reshape(1, M, D)
    W1 = torch.empty(N, D, 2 * H, device=DEV, dtype=torch.bfloat16).normal_(0, 0.02, generator=gen)
    W2 = torch.empty(N, H, D, device=DEV, dtype=torch.bfloat16).normal_(0, 0.02, generator=gen)
    mask, s = routing(M, N, K, Ks, skew, gen)
    layer = momoe_amd.MoMoE(D, H, N, K, sp, Wl1_ND2H=W1, Wl2_NHD=W2)

    def fwd():
        with torch.no_grad():
            layer(x, mask, s)

    def step():
        xd, sd = x.detach().requires_grad_(), s.detach().requires_grad_()
        y, _ = layer(xd, mask, sd)
        y.backward(dy)
        layer.Wl1_ND2H.grad = layer.Wl2_NHD.grad = None

    def timeit(fn):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e3

    unit = float(D) * H * M * K
    tf = timeit(fwd)
    line = f"{name:30s} fwd {tf:8.3f} ms {6 * unit / tf / 1e9:6.0f} TF/s {M / tf * 1e3:11.0f} tok/s"
    if graph:
        # the same call captured once in a HIP graph and replayed: what a serving loop pays per
        # call when the host does not launch kernel by kernel (no launch is sized from the routing
        # on the host, so the replay stays valid when mask and gate weights change in place)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fwd()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            fwd()
        tg = timeit(g.replay)
        line += f" | graph replay {tg:8.3f} ms {M / tg * 1e3:11.0f} tok/s"
        del g
    if backward:
        torch.cuda.reset_peak_memory_stats()
        tb = timeit(step)
        line += (f" | fwd+bwd {tb:8.3f} ms {18 * unit / tb / 1e9:6.0f} TF/s {M / tb * 1e3:10.0f} tok/s"
                 f" | peak {torch.cuda.max_memory_allocated() / 2**30:5.2f} GiB")
    print(line, flush=True)


def chart_row(B, S, D, H, N, K, kind, steps=5):
    """One configuration of the reference's charts: forward TF/s, forward+backward TF/s at
    save_percent 0 / 50 / 100 and, per save_percent, the bytes alive after forward that were
    not alive before it plus x itself (what the reference's memory chart plots: x, y and the
    tensors saved for backward; weights, mask and gates excluded)."""
    M = B * S
    gen = torch.Generator(device=DEV).manual_seed(1)
    x = torch.randn(M, D, generator=gen, device=DEV).to(torch.bfloat16).reshape(B, S, D)
    dy = torch.randn(M, D, generator=gen, device=DEV).to(torch.bfloat16).reshape(B, S, D)
    W1 = torch.empty(N, D, 2 * H, device=DEV, dtype=torch.bfloat16).normal_(0, 0.02, generator=gen)
    W2 = torch.empty(N, H, D, device=DEV, dtype=torch.bfloat16).normal_(0, 0.02, generator=gen)
    if kind == "balanced":
        mask, s = balanced_routing(M, N, K, gen)
    else:
        mask, s = routing(M, N, K, 0, 1.8 if kind == "skewed" else None, gen)
    unit = float(D) * H * M * K
    cells, result = [], {}
    for sp in (0, 50, 100):
        layer = momoe_amd.MoMoE(D, H, N, K, sp, Wl1_ND2H=W1, Wl2_NHD=W2)

        def fwd():
            with torch.no_grad():
                layer(x, mask, s)

        def step(measure=False):
            xd, sd = x.detach().requires_grad_(), s.detach().requires_grad_()
            before = torch.cuda.memory_allocated()
            y, _ = layer(xd, mask, sd)
            held = torch.cuda.memory_allocated() - before + x.numel() * 2
            y.backward(dy)
            del y
            layer.Wl1_ND2H.grad = layer.Wl2_NHD.grad = None
            return held

        def timeit(fn):
            for _ in range(2):
                fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                fn()
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) / steps * 1e3

        tf, tb = timeit(fwd), timeit(step)
        held = step()
        result[sp] = {"fwd_tflops": 6 * unit / tf / 1e9, "fwd_bwd_tflops": 18 * unit / tb / 1e9,
                      "held_bytes": held}
        cells.append(f"sp{sp:3d}: fwd {6 * unit / tf / 1e9:5.0f} f+b {18 * unit / tb / 1e9:5.0f} TF/s"
                     f" held {held / 1e9:5.2f} GB")
        del layer
    print(f"{B},{S},{D},{H},{N},{K} {kind:8s} | " + " | ".join(cells), flush=True)
    return result


def vendor_gemms(D=2048, H=1024, N=128, R=512, steps=20):
    """What the vendor GEMM library (torch.bmm) gives the two forward GEMMs of a step on this
    machine when every expert holds exactly R rows: no gather, no epilogue, no ragged tiles,
    outputs in bf16.  The figures to read this library's per-kernel times against (bench.py
    `kernels`): the same products on the same data distribution, N(0,1) activations and
    N(0,0.02) weights.
    Only the products with untransposed operands are timed.  The transposed ones (the data and
    weight gradients) are left out on purpose: on this image the batched product
    gz[128,512,2048] . Wl1[128,2048,2048]^T ends in an illegal memory access inside the vendor
    library (no kernel of this repository involved) and takes the GPU down with it."""
    gen = torch.Generator(device=DEV).manual_seed(0)
    rnd = lambda *shape: torch.randn(*shape, generator=gen, device=DEV).to(torch.bfloat16)
    x, h = rnd(N, R, D), rnd(N, R, H)
    W1, W2 = rnd(N, D, 2 * H) * 0.02, rnd(N, H, D) * 0.02
    unit = float(D) * H * R * N
    cases = [
        ("momoe_lin1_swiglu_fwd", f"x[{R},{D}] . Wl1[{D},{2 * H}]", 4, lambda: torch.bmm(x, W1)),
        ("momoe_lin2_scale_fwd", f"h[{R},{H}] . Wl2[{H},{D}]", 2, lambda: torch.bmm(h, W2)),
    ]
    print(f"torch.bmm over {N} experts of {R} rows each, bf16; ms per call and TFLOP/s", flush=True)
    out = {}
    for name, shape, units, fn in cases:
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / steps
        out[name] = ms
        print(f"{name:24s} {shape:36s} {ms:7.3f} ms {units * unit / ms / 1e9:6.0f} TF/s", flush=True)
    return out


def read_stream_rate(gib=1.5):
    """GB/s at which the weight stream of the grouped GEMMs alone (global -> LDS transfers, nothing
    else: momoe_hbm_stream_probe) reads a tensor larger than the 256 MiB last-level cache.  The
    figure to read the weight-streaming GEMMs of the decode-sized calls against: it is what this
    machine delivers to that access pattern, whatever the 8 TB/s of the data sheet say."""
    blocks = int(gib * 2**30) // (2048 * 2048 * 2)
    w = torch.empty((blocks, 2048, 2048), dtype=torch.bfloat16, device=DEV).normal_()
    rate = _hip.hbm_stream_probe(w)
    print(f"weight stream alone over {blocks * 8} MiB: {rate:7.0f} GB/s", flush=True)
    return rate


CHART_GRID = [
    (2, 512, 1024, 512, 32, 4, "balanced"), (4, 2048, 2048, 1024, 64, 8, "balanced"),
    (4, 2048, 2048, 1024, 64, 8, "skewed"), (6, 2048, 2048, 1280, 64, 6, "balanced"),
    (4, 1920, 2176, 1152, 64, 6, "random"), (8, 4096, 2048, 1024, 128, 8, "balanced"),
    (8, 4096, 2048, 1024, 128, 8, "skewed"), (8, 8192, 2048, 1024, 128, 8, "balanced"),
]


if __name__ == "__main__":
    assert torch.cuda.is_available() and _hip.abi_version() == 3
    if "--vendor" in sys.argv[1:]:
        vendor_gemms()
        read_stream_rate()
        sys.exit(0)
    if "--chart" in sys.argv[1:]:
        for row in CHART_GRID:
            chart_row(*row)
        sys.exit(0)
    only = sys.argv[sys.argv.index("--only") + 1] if "--only" in sys.argv[1:] else None
    if only in (None, "inference"):
        for M in (16, 128, 1024, 8192):
            run(f"inference D2048 H768, M={M}", M, 2048, 768, 128, 8, backward=False, steps=20, graph=True)
    if only in (None, "headline"):
        run("headline D2048 H1024", 8192, 2048, 1024, 128, 8)
    if only in (None, "skewed"):
        run("skewed + 4 shared, H1408", 16384, 2048, 1408, 64, 8, Ks=4, skew=1.5 * 1.2)
    if only in (None, "large"):
        for sp in (0, 50, 100):
            run(f"D4096 H2048, save_percent={sp}", 65536, 4096, 2048, 64, 8, sp=sp, steps=3)
