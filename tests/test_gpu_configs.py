"""GPU: the benchmark plan's remaining configurations at their full sizes -- the Qwen3-shaped
inference forward (D=2048, H=768, N=128, K=8, no autograd) over the decode-to-prefill token
sweep -- the memory contract of the layer, and a routing that breaks the "exactly K experts per
token" precondition."""
import pytest
import torch

import oracle
from gpu_util import (assert_close, device_layer_inputs, oracle_forward_for_tokens, run_device_layer,
                      run_oracle_layer)
from helpers import make_layer_inputs

pytestmark = pytest.mark.gpu

MiB = 2**20


@pytest.mark.parametrize("M", [16, 128, 1024, 8192])
def test_inference_forward_sweep(M):
    # forward only under torch.no_grad() (momoe/momoe.py:244-290).  16 and 128 tokens: every
    # token against the oracle; 1024 and 8192: a sample of 32 tokens (each with all of its 8
    # experts) plus the tokens-per-expert histogram and size-independent properties.
    import momoe_amd
    D, H, N, K = 2048, 768, 128, 8
    dev = "cuda:0"
    x, _, W1, W2, mask, s = device_layer_inputs(M, D, H, N, K, seed=31, routing_seed=M)
    layer = momoe_amd.MoMoE(D, H, N, K, save_percent=100, Wl1_ND2H=W1, Wl2_NHD=W2)
    maskd, sd = mask.to(dev), s.T.contiguous().to(dev).T
    xb = x.reshape(1, M, D)
    with torch.no_grad():
        y, sizes = layer(xb, maskd, sd)
        y2, _ = layer(xb, maskd, 2 * sd)
    torch.cuda.synchronize()
    assert y.dtype == torch.bfloat16 and y.shape == (1, M, D) and not y.requires_grad
    assert sizes.dtype == torch.int64 and torch.equal(sizes.cpu(), (mask != 0).sum(1))
    assert torch.isfinite(y).all()
    tok = torch.arange(M) if M <= 128 else torch.arange(0, M, M // 32)[:32]
    yo, _ = oracle_forward_for_tokens(x, W1, W2, mask, s, tok)
    assert_close(y.reshape(M, D)[tok.to(dev)], yo, f"y, {M} tokens")
    # linear in the gate weights, up to the bf16 rounding of y
    from gpu_util import rel_err
    assert rel_err(y2, 2 * y) < 5e-3


def test_no_grad_forward_keeps_and_allocates_nothing_for_a_backward():
    # save_percent=100 under no_grad must not write or hold the pre-activations: same peak and
    # same memory afterwards as save_percent=0
    import momoe_amd
    M, D, H, N, K = 4096, 1024, 512, 32, 4
    dev = "cuda:0"
    x, dy, W1, W2, mask, s = device_layer_inputs(M, D, H, N, K)
    maskd, sd, xb = mask.to(dev), s.T.contiguous().to(dev).T, x.reshape(1, M, D)
    peaks, helds = [], []
    for sp in (0, 100):
        layer = momoe_amd.MoMoE(D, H, N, K, save_percent=sp, Wl1_ND2H=W1, Wl2_NHD=W2)
        torch.cuda.synchronize()
        base = torch.cuda.memory_allocated()
        torch.cuda.reset_peak_memory_stats()
        with torch.no_grad():
            y, sizes = layer(xb, maskd, sd)
        torch.cuda.synchronize()
        peaks.append(torch.cuda.max_memory_allocated() - base)
        helds.append(torch.cuda.memory_allocated() - base - y.numel() * 2)
        del y, sizes, layer
    assert peaks[0] == peaks[1] and helds[0] == helds[1]
    assert helds[0] < 64 * 1024  # only the tokens-per-expert vector outlives the call


@pytest.mark.parametrize("M,D,H,N,K", [(8192, 2048, 1024, 128, 8)])
def test_memory_contract_at_the_headline_layer(M, D, H, N, K):
    # The reference's allocation sites (momoe/momoe.py:252-257, 550-556, 720-722, 872) give, at
    # save_percent=0: forward transient h + y_KMD + y = Msum*H*2 + K*M*D*2 + M*D*2 bytes (416 MiB
    # here); backward transient x_MsumD + G_z + h + G_x_KMD + G_s + G_x = 932 MiB on top of the
    # weight gradients; held between forward and backward: the routing index only.  This build
    # must not exceed any of them, and what it holds must not shrink as save_percent grows.
    # The 2 MiB of slack covers the routing index and its scratch (idx, inv, which, the tile
    # list; the reference's idx / which / counters are not in its 416 MiB either).
    import momoe_amd
    dev = "cuda:0"
    msum = M * K
    fwd_budget = msum * H * 2 + K * M * D * 2 + M * D * 2
    bwd_budget = msum * D * 2 + msum * 2 * H * 2 + msum * H * 2 + K * M * D * 2 + N * M * 4 + M * D * 2
    assert fwd_budget == 416 * MiB and bwd_budget == 932 * MiB
    wgrad_bytes = N * D * 2 * H * 2 + N * H * D * 2
    x, dy, W1, W2, mask, s = device_layer_inputs(M, D, H, N, K)
    maskd = mask.to(dev)
    held = {}
    for sp in (0, 50, 100):
        layer = momoe_amd.MoMoE(D, H, N, K, save_percent=sp, Wl1_ND2H=W1, Wl2_NHD=W2)
        xd = x.reshape(4, M // 4, D).clone().requires_grad_()
        sd = s.T.contiguous().to(dev).T.requires_grad_()
        dyd = dy.reshape(4, M // 4, D)
        torch.cuda.synchronize()
        base = torch.cuda.memory_allocated()
        torch.cuda.reset_peak_memory_stats()
        y, _ = layer(xd, maskd, sd)
        torch.cuda.synchronize()
        fwd_peak = torch.cuda.max_memory_allocated() - base
        held[sp] = torch.cuda.memory_allocated() - base - y.numel() * 2
        y.backward(dyd)
        torch.cuda.synchronize()
        total_peak = torch.cuda.max_memory_allocated() - base
        saved = int(msum * sp / 100.0) * 2 * H * 2
        print(f"[memory] save_percent={sp}: forward peak {fwd_peak / MiB:.1f} MiB, held {held[sp] / MiB:.2f} MiB, "
              f"fwd+bwd peak without weight gradients {(total_peak - wgrad_bytes) / MiB:.1f} MiB")
        assert fwd_peak <= fwd_budget + saved + 2 * MiB
        # y (the caller's) and the saved pre-activations stay alive through the backward
        assert total_peak - wgrad_bytes <= bwd_budget + saved + 2 * MiB
        # what is held is the routing index plus exactly the saved a|b rows
        assert saved <= held[sp] <= saved + 1 * MiB
        del layer, xd, sd, y
    assert held[0] < 1 * MiB
    assert held[0] <= held[50] <= held[100]
    # the reference holds a, b AND y_pre for the saved rows (momoe/momoe.py:252-255)
    assert held[100] <= msum * (2 * H + D) * 2 + 1 * MiB


@pytest.mark.parametrize("sp", [0, 100])
def test_tokens_with_fewer_than_k_experts(sp):
    # The layer's precondition is exactly K experts per token (momoe/momoe.py:831).  With fewer,
    # the sorted rows past the last pair do not exist: nothing may read an undefined token id,
    # and the result is the sum over the pairs that do exist -- which is what the oracle computes.
    M, D, H, N, K = 300, 128, 96, 8, 3
    x, W1, W2, mask, s, dy = make_layer_inputs(M, D, H, N, K, seed=4)
    mask = mask.clone()
    s = s.clone()
    for m in (0, 7, 150, 299):        # these tokens lose their lowest-numbered expert
        i = int(torch.nonzero(mask[:, m])[0])
        mask[i, m] = 0
        s[i, m] = 0.0
    mask[:, 42] = 0                   # and one token has no expert at all
    s[:, 42] = 0.0
    dev = run_device_layer(x, W1, W2, mask, s, dy, K, sp)
    ref = run_oracle_layer(x, W1, W2, mask, s, dy)
    assert torch.equal(dev["sizes"], ref["sizes"])
    for k in ("y", "G_x", "G_W1", "G_W2", "G_s"):
        assert_close(dev[k], ref[k], k)
    assert torch.all(dev["y"][42] == 0) and torch.all(dev["G_x"][42] == 0)


@pytest.mark.parametrize("M,sp", [(300, 0), (300, 100), (2000, 50)])
def test_mask_with_more_than_mk_pairs_gives_zeros(M, sp):
    # More pairs than sorted rows exist for: the routing is refused on the device (empty tile
    # table, violation counted).  No GEMM runs, and what is returned is defined all the same:
    # y and every gradient are zero, never unwritten memory.
    import momoe_amd
    D, H, N, K = 128, 96, 8, 3
    x, W1, W2, mask, s, dy = make_layer_inputs(M, D, H, N, K, seed=6)
    mask = mask.clone()
    mask[:, ::2] = 1                  # every second token sits on all experts
    s = torch.rand(N, M) * mask
    dev = "cuda:0"
    # poison the allocator's free blocks, which the layer's torch.empty buffers will reuse
    junk = torch.full((64 * 2**20,), float("nan"), device=dev, dtype=torch.bfloat16)
    del junk
    layer = momoe_amd.MoMoE(D, H, N, K, save_percent=sp, Wl1_ND2H=W1.to(dev), Wl2_NHD=W2.to(dev))
    xd = x.to(dev, torch.bfloat16).reshape(1, M, D).requires_grad_()
    sd = s.to(dev).requires_grad_()
    y, sizes = layer(xd, mask.to(dev), sd)
    y.backward(dy.to(dev, torch.bfloat16).reshape(1, M, D))
    torch.cuda.synchronize()
    assert torch.equal(sizes.cpu(), (mask != 0).sum(1))
    for t in (y, xd.grad, layer.Wl1_ND2H.grad, layer.Wl2_NHD.grad, sd.grad):
        assert torch.all(t == 0)


def test_opt_in_routing_check_raises():
    import momoe_amd
    from momoe_amd import experts
    M, D, H, N, K = 64, 64, 32, 4, 2
    x, W1, W2, mask, s, _ = make_layer_inputs(M, D, H, N, K, seed=5)
    mask = mask.clone()
    mask[:, 3] = 0
    layer = momoe_amd.MoMoE(D, H, N, K, Wl1_ND2H=W1.cuda(), Wl2_NHD=W2.cuda())
    experts.CHECK_ROUTING = True
    try:
        with pytest.raises(RuntimeError, match="exactly K"):
            layer(x.cuda().reshape(1, M, D), mask.cuda(), s.cuda())
        good, sg = make_layer_inputs(M, D, H, N, K, seed=5)[3:5]
        layer(x.cuda().reshape(1, M, D), good.cuda(), sg.cuda())
    finally:
        experts.CHECK_ROUTING = False


def test_chart_grid_harness_one_cell():
    # the harness behind the README-chart table (momoe-impl_amd/bench_configs.py --chart): run its
    # smallest cell (B=2, S=512, D=1024, H=512, N=32, K=4, balanced routing) and check what it
    # reports is sane: positive rates, the memory held between forward and backward equal to
    # x + y + routing index at save_percent=0 and growing by the saved a|b rows
    import bench_configs
    B, S, D, H, N, K = bench_configs.CHART_GRID[0][:6]
    res = bench_configs.chart_row(*bench_configs.CHART_GRID[0], steps=2)
    M = B * S
    xy = 2 * M * D * 2
    for sp in (0, 50, 100):
        assert res[sp]["fwd_tflops"] > 1 and res[sp]["fwd_bwd_tflops"] > 1
        saved = int(M * K * sp / 100.0) * 2 * H * 2
        assert xy + saved <= res[sp]["held_bytes"] <= xy + saved + MiB


@pytest.mark.parametrize("M,N,K", [(12288, 64, 6), (1000, 7, 3), (64, 64, 8)])
def test_balanced_routing_of_the_chart_harness(M, N, K):
    # the "balanced" cells of the chart grid include one whose K does not divide N
    # (6 x 2048 tokens, N=64, K=6): every token still gets K distinct experts and every expert
    # floor(M*K/N) or ceil(M*K/N) tokens
    import bench_configs
    gen = torch.Generator(device="cuda:0").manual_seed(0)
    mask, s = bench_configs.balanced_routing(M, N, K, gen)
    mask, s = mask.cpu(), s.cpu()
    assert mask.shape == (N, M) and torch.all(mask.sum(0) == K)
    sizes = mask.sum(1)
    assert sizes.min() >= (M * K) // N and sizes.max() <= -(-(M * K) // N)
    assert torch.allclose(s.sum(0), torch.ones(M), atol=1e-5) and torch.all(s[mask == 0] == 0)


@pytest.mark.parametrize("sp", [0, 50])
def test_layer_under_hip_graph_replay(sp):
    """The whole forward+backward of the layer captured once in a HIP graph (torch.cuda.CUDAGraph)
    and replayed on new inputs and new routings: no launch is sized from the routing on the host
    and nothing synchronises, so the captured launches stay valid.  Every replay is checked against
    the eager result (bit-identical), with eager work and synchronisations between the replays."""
    import momoe_amd
    M, D, H, N, K = 1024, 256, 160, 16, 4
    dev = "cuda:0"

    def inputs(seed):
        x, W1, W2, mask, s, dy = make_layer_inputs(M, D, H, N, K, seed=seed, skew=1.0 if seed % 2 else None)
        return (x.to(dev, torch.bfloat16).reshape(1, M, D), mask.to(dev), s.to(dev),
                dy.to(dev, torch.bfloat16).reshape(1, M, D), W1.to(dev), W2.to(dev))

    x0, mask0, s0, dy0, W1, W2 = inputs(40)
    layer = momoe_amd.MoMoE(D, H, N, K, save_percent=sp, Wl1_ND2H=W1, Wl2_NHD=W2)
    sx, smask, ss, sdy = x0.clone().requires_grad_(), mask0.clone(), s0.clone().requires_grad_(), dy0.clone()

    def step(x, mask, s, dy):
        for t in (x, s, layer.Wl1_ND2H, layer.Wl2_NHD):
            t.grad = None
        y, sizes = layer(x, mask, s)
        y.backward(dy)
        return y.detach(), sizes, x.grad, s.grad, layer.Wl1_ND2H.grad, layer.Wl2_NHD.grad

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):  # warm-up outside the capture (first-call set-up of the library included)
            step(sx, smask, ss, sdy)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step(sx, smask, ss, sdy)
    for seed in (41, 42, 43, 40):
        x, mask, s, dy, _, _ = inputs(seed)
        eager = [t.clone() for t in step(x.clone().requires_grad_(), mask, s.clone().requires_grad_(), dy)]
        torch.cuda.synchronize()
        with torch.no_grad():
            sx.copy_(x); smask.copy_(mask); ss.copy_(s); sdy.copy_(dy)
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("y", "sizes", "G_x", "G_s", "G_W1", "G_W2"), captured, eager):
            assert torch.equal(a, b), (seed, name)


def test_measurement_aids_of_the_benchmark():
    # bench.py runs the layer under the in-kernel clock trace and the per-launch timer, and
    # times the bare MFMA loop: the same calls at a small size, with plausible results
    # (a shader clock between 0.5 and 3 GHz, every entry point of a step timed once per step,
    # an MFMA rate above a tenth of the published peak).
    import momoe_amd
    from momoe_amd import _hip
    M, D, H, N, K = 2048, 512, 256, 16, 4
    dev = "cuda:0"
    x, dy, W1, W2, mask, s = device_layer_inputs(M, D, H, N, K)
    layer = momoe_amd.MoMoE(D, H, N, K, save_percent=0, Wl1_ND2H=W1, Wl2_NHD=W2)
    maskd = mask.to(dev)

    def step():
        xd = x.reshape(1, M, D).clone().requires_grad_()
        sd = s.T.contiguous().to(dev).T.requires_grad_()
        y, _ = layer(xd, maskd, sd)
        y.backward(dy.reshape(1, M, D))
        layer.Wl1_ND2H.grad = layer.Wl2_NHD.grad = None
        return y

    ref = step()
    with _hip.clock_trace() as ct, _hip.kernel_timer() as kt:
        for _ in range(4):
            got = step()
    mhz = ct.mhz()
    names = [n for n, _ in kt.durations_ms()]
    assert 500 < mhz < 3000, mhz
    for entry in ("momoe_index_build", "momoe_lin1_swiglu_fwd", "momoe_lin2_scale_fwd", "momoe_dgrad_h",
                  "momoe_lin1_swiglu_bwd", "momoe_dgrad_x", "momoe_gs_scatter"):
        assert names.count(entry) == 4, (entry, names.count(entry))
    assert names.count("momoe_wgrad") == 8 and names.count("momoe_combine") == 8
    assert torch.equal(got, ref)   # tracing changes no result
    tf, clk = _hip.mfma_rate_probe("zeros", iters=2000, launches=2)
    assert tf > 250 and 500 < clk < 3000, (tf, clk)


def test_backward_row_limit_is_reported_in_the_forward():
    # the Wl1 gradient takes fewer than 8 388 608 (token, expert) pairs per call (32-bit offsets
    # into the k-blocked gz): a larger training batch is refused before anything is launched,
    # not in the backward after the forward succeeded
    import momoe_amd
    D, H, N, K = 32, 32, 8, 8
    M = 2 ** 20
    dev = "cuda:0"
    layer = momoe_amd.MoMoE(D, H, N, K)
    x = torch.zeros(1, M, D, device=dev, dtype=torch.bfloat16)
    mask = torch.ones(N, M, device=dev, dtype=torch.int32)
    s = torch.full((N, M), 1.0 / N, device=dev)
    with pytest.raises(RuntimeError, match="8388608"):
        layer(x, mask, s)
    del x, mask, s
