"""GPU: MoMoE forward + backward through the C ABI against the CPU oracle on the same
seeded inputs.  Tolerance: rtol 2e-2 / atol 2e-2 (bf16 results vs fp32-accumulated
oracle) plus a norm-wise bound; tokens-per-expert bit-exact."""
import pytest
import torch

import oracle
from gpu_util import (assert_close, rel_err, run_device_layer, run_oracle_layer,
                      sampled_parity_on_device_inputs as _sampled_parity_on_device_inputs)
from helpers import make_layer_inputs

pytestmark = pytest.mark.gpu


def _check_all(dev, ref, rel=1e-2):
    assert torch.equal(dev["sizes"], ref["sizes"])
    for k in ("y", "G_x", "G_W1", "G_W2", "G_s"):
        assert_close(dev[k], ref[k], k, rel=rel)


@pytest.mark.parametrize("save_percent", [0, 50, 100])
def test_tiny_reference_config(save_percent):
    # B=2, S=64, D=128, H=64, N=8, K=2
    M, D, H, N, K = 128, 128, 64, 8, 2
    x, W1, W2, mask, s, dy = make_layer_inputs(M, D, H, N, K, seed=0)
    dev = run_device_layer(x, W1, W2, mask, s, dy, K, save_percent, B=2)
    ref = run_oracle_layer(x, W1, W2, mask, s, dy)
    _check_all(dev, ref)
    assert dev["y"].dtype == torch.bfloat16 and dev["G_s"].dtype == torch.float32
    assert dev["G_W1"].dtype == torch.bfloat16 and dev["G_x"].dtype == torch.bfloat16
    assert torch.all(dev["G_s"][mask == 0] == 0)


@pytest.mark.parametrize("M,D,H,N,K,Ks,skew,sp", [
    (1024, 512, 256, 16, 4, 0, None, 0),
    (1024, 512, 256, 16, 4, 0, None, 37),    # save boundary in the middle of a tile
    (999, 256, 320, 12, 3, 0, None, 100),    # ragged token count, H not a multiple of the column tile
    (2048, 512, 384, 20, 6, 2, 1.8, 0),      # skew + shared experts, H = 1.5 column tiles
    (2048, 512, 384, 20, 6, 2, 1.8, 100),
    (16, 256, 128, 32, 4, 0, None, 0),       # decode-sized: most experts empty
    (64, 64, 32, 1, 1, 0, None, 0),          # one expert, smallest supported D and H
    (33, 96, 160, 5, 5, 0, None, 50),        # every token on every expert, odd token count
    (700, 160, 96, 3, 2, 1, None, 0),        # experts taller than one tile, one shared expert
    (9000, 64, 96, 3, 2, 1, None, 0),        # a shared expert with enough rows that its weight
                                             # gradient is contracted in several pieces
    (12000, 96, 64, 6, 1, 0, 1.8, 50),       # one routed expert holds most rows
])
def test_layer_parity(M, D, H, N, K, Ks, skew, sp):
    x, W1, W2, mask, s, dy = make_layer_inputs(M, D, H, N, K, Ks=Ks, seed=5, skew=skew)
    dev = run_device_layer(x, W1, W2, mask, s, dy, K, sp)
    ref = run_oracle_layer(x, W1, W2, mask, s, dy)
    _check_all(dev, ref)


@pytest.mark.parametrize("seed", range(16))
def test_random_small_shapes(seed):
    # shapes drawn from a seeded generator: odd token counts, D and H any multiple of 32,
    # few or many experts, shared experts, every save_percent regime
    import random
    rng = random.Random(1000 + seed)
    D, H = 32 * rng.randint(1, 10), 32 * rng.randint(1, 10)
    N = rng.randint(1, 40)
    K = rng.randint(1, min(N, 6))
    Ks = rng.randint(0, K - 1) if rng.random() < 0.4 else 0
    M = rng.choice([1, 7, 64, 255, 256, 257, 600, 901])
    sp = rng.choice([0, 0, 25, 50, 100])
    skew = rng.choice([None, None, 1.5])
    x, W1, W2, mask, s, dy = make_layer_inputs(M, D, H, N, K, Ks=Ks, seed=seed, skew=skew)
    dev = run_device_layer(x, W1, W2, mask, s, dy, K, sp)
    ref = run_oracle_layer(x, W1, W2, mask, s, dy)
    _check_all(dev, ref)
    # the same through the 320-row code path of the forward and data-gradient GEMMs, which small
    # routings never choose by themselves: bit-identical to the run above
    from momoe_amd import _hip, experts
    try:
        experts.TILE_ROWS = _hip.TILE_ROWS
        tall = run_device_layer(x, W1, W2, mask, s, dy, K, sp)
    finally:
        experts.TILE_ROWS = _hip.AUTO_TILE_ROWS
    for k in dev:
        assert torch.equal(tall[k], dev[k]), k


@pytest.mark.parametrize("gather_a", [True, False])
def test_weight_gradient_of_cut_experts(gather_a):
    # experts of 20000 / 3 / 0 / 5000 rows: the first is contracted in pieces that meet in the
    # fp32 workspace.  Checked against a plain fp32 matmul per expert and against the same
    # launch without a workspace (no expert is cut then).
    from momoe_amd import _hip
    dev = "cuda:0"
    sizes = [20000, 3, 0, 5000]
    N, X, Y, M = len(sizes), 320, 512, 20000
    msum = sum(sizes)
    g = torch.Generator(device=dev).manual_seed(11)
    cumsums = torch.tensor([0] + list(torch.tensor(sizes).cumsum(0)), dtype=torch.int32, device=dev)
    A = torch.randn(M if gather_a else msum, X, generator=g, device=dev).to(torch.bfloat16)
    B = torch.randn(msum if gather_a else M, Y, generator=g, device=dev).to(torch.bfloat16)
    ids = torch.cat([torch.randperm(M, generator=g, device=dev)[:n].sort().values for n in sizes]).to(torch.int32)
    ga, gb = (ids, None) if gather_a else (None, ids)
    need = _hip._lib.momoe_wgrad_workspace_bytes(N, X, Y, msum)
    assert need >= 3 * 4 * 262144
    out = {}
    for ws in (need, 262144 * 16, 0):
        GW = torch.full((N, X, Y), float("nan"), device=dev, dtype=torch.bfloat16)
        _hip.wgrad(A, ga, B, gb, cumsums, GW, M, msum, workspace_bytes=ws)
        out[ws] = GW.float()
    torch.cuda.synchronize()
    for e, n in enumerate(sizes):
        r0 = int(cumsums[e])
        Ae = A[ids[r0:r0 + n].long()] if gather_a else A[r0:r0 + n]
        Be = B[r0:r0 + n] if gather_a else B[ids[r0:r0 + n].long()]
        want = Ae.float().T @ Be.float()
        for ws, got in out.items():
            assert_close(got[e].cpu(), want.cpu(), f"GW[{e}] ws={ws}", rel=5e-3)
    assert torch.equal(out[0][2], torch.zeros(X, Y, device=dev))
    assert torch.equal(out[need][1:3], out[0][1:3])  # uncut experts: bit-identical


@pytest.mark.parametrize("sizes,M", [([300, 0, 17, 1000, 64], 1000), ([20000, 3, 0, 5000], 20000)])
def test_weight_gradient_from_a_transposed_operand(sizes, M):
    # either operand handed over as [padded sorted row / 32, feature, 32] (the layout the SwiGLU
    # backward writes s*h in): same result as from the row layout, against a plain fp32 matmul
    from momoe_amd import _hip
    dev = "cuda:0"
    N, X, Y = len(sizes), 320, 512
    msum = sum(sizes)
    g = torch.Generator(device=dev).manual_seed(5)
    c = [0] + list(torch.tensor(sizes).cumsum(0).tolist())
    cumsums = torch.tensor(c, dtype=torch.int32, device=dev)
    A = torch.randn(msum, X, generator=g, device=dev).to(torch.bfloat16)
    B = torch.randn(msum, Y, generator=g, device=dev).to(torch.bfloat16)

    def grouped(rows):
        F = rows.shape[1]
        mpad = _hip.padded_rows(msum, N)
        assert mpad == (msum + 31) // 32 * 32 + 32 * N
        # garbage outside the experts' own 32-row groups must not matter; zeros inside them do
        T = torch.full((F, mpad), float("nan"), device=dev, dtype=rows.dtype)
        for e in range(N):
            p0 = (c[e] + 31) // 32 * 32 + 32 * e
            n = c[e + 1] - c[e]
            T[:, p0:p0 + (n + 31) // 32 * 32] = 0
            T[:, p0:p0 + n] = rows[c[e]:c[e + 1]].T
        return T.reshape(F, mpad // 32, 32).permute(1, 0, 2).contiguous()

    # k-blocked B: [feature / 32, row, 32]
    blocked_B = B.reshape(msum, Y // 32, 32).permute(1, 0, 2).contiguous()
    want = torch.stack([A[c[e]:c[e + 1]].float().T @ B[c[e]:c[e + 1]].float() for e in range(N)])
    for kw, a, b in ((dict(a_transposed=True), grouped(A), B), (dict(b_transposed=True), A, grouped(B)),
                     (dict(b_kblocked=True), A, blocked_B)):
        for ws in (None, 0):
            GW = torch.full((N, X, Y), float("nan"), device=dev, dtype=torch.bfloat16)
            _hip.wgrad(a, None, b, None, cumsums, GW, M, msum, workspace_bytes=ws, **kw)
            torch.cuda.synchronize()
            for e in range(N):
                assert_close(GW[e], want[e], f"GW[{e}] {kw} ws={ws}", rel=5e-3)
    with pytest.raises(RuntimeError):  # both transposed: refused
        _hip.wgrad(grouped(A), None, grouped(B), None, cumsums, GW, M, msum, a_transposed=True, b_transposed=True)


def test_experts_without_tokens_get_zero_weight_grads():
    M, D, H, N, K = 256, 128, 64, 8, 2
    x, W1, W2, _, _, dy = make_layer_inputs(M, D, H, N, K, seed=9)
    mask = torch.zeros(N, M, dtype=torch.int32)
    mask[1] = 1
    mask[6] = 1
    s = torch.rand(N, M) * mask
    dev = run_device_layer(x, W1, W2, mask, s, dy, K, 0)
    ref = run_oracle_layer(x, W1, W2, mask, s, dy)
    _check_all(dev, ref)
    for i in (0, 2, 3, 4, 5, 7):
        assert torch.all(dev["G_W1"][i] == 0) and torch.all(dev["G_W2"][i] == 0)


def test_save_percent_only_changes_rounding():
    M, D, H, N, K = 2048, 512, 256, 16, 4
    x, W1, W2, mask, s, dy = make_layer_inputs(M, D, H, N, K, seed=12)
    r0 = run_device_layer(x, W1, W2, mask, s, dy, K, 0)
    r100 = run_device_layer(x, W1, W2, mask, s, dy, K, 100)
    assert torch.equal(r0["y"], r100["y"])  # forward does not depend on what is saved
    for k in ("G_x", "G_W1", "G_W2", "G_s"):
        assert rel_err(r0[k], r100[k]) < 1e-2, k


def test_headline_shape_properties_and_sampled_parity():
    # Full headline layer: D=2048, H=1024, N=128, K=8, 8192 tokens.  The oracle is evaluated
    # on a sample of tokens / experts; size-independent properties cover the rest.
    import momoe_amd
    M, D, H, N, K = 8192, 2048, 1024, 128, 8
    x, W1, W2, mask, s, dy = make_layer_inputs(M, D, H, N, K, seed=21)
    dev = "cuda:0"
    layer = momoe_amd.MoMoE(D, H, N, K, 0, Wl1_ND2H=W1.to(dev), Wl2_NHD=W2.to(dev))
    xd = x.to(dev, torch.bfloat16).reshape(4, 2048, D).requires_grad_()
    sd = s.T.contiguous().to(dev).T.requires_grad_()
    y, sizes = layer(xd, mask.to(dev), sd)
    y.backward(dy.to(dev, torch.bfloat16).reshape(4, 2048, D))
    torch.cuda.synchronize()
    assert sizes.sum().item() == M * K and torch.equal(sizes.cpu(), (mask != 0).sum(1))
    assert torch.isfinite(y).all() and torch.isfinite(layer.Wl1_ND2H.grad).all()
    # linearity in the gate weights: y(2s) == 2*y(s) up to bf16 rounding
    with torch.no_grad():
        y2, _ = layer(xd, mask.to(dev), 2 * sd)
    assert rel_err(y2, 2 * y) < 5e-3
    # sampled forward parity: 48 tokens, all of their experts
    r = lambda t: t.to(torch.bfloat16).float()
    tok = torch.arange(0, M, M // 48)[:48]
    yo = oracle.experts_forward(r(x[tok]), r(W1), r(W2), mask[:, tok], s[:, tok])
    assert_close(y.reshape(M, D)[tok], yo, "y (sampled tokens)")
    # sampled weight-gradient / dL/ds parity: experts 0, 77 and 127 from the closed form
    for i in (0, 77, 127):
        sel = torch.nonzero(mask[i]).flatten()
        one = torch.zeros(1, sel.numel(), dtype=torch.int32) + 1
        _, gW1, gW2, gs = oracle.experts_backward_closed_form(
            r(x[sel]), r(W1[i:i + 1]), r(W2[i:i + 1]), one, s[i:i + 1, sel], r(dy[sel]), dtype=torch.float32)
        assert_close(layer.Wl1_ND2H.grad[i], gW1[0], f"G_W1[{i}]")
        assert_close(layer.Wl2_NHD.grad[i], gW2[0], f"G_W2[{i}]")
        assert_close(sd.grad[i, sel], gs[0], f"G_s[{i}]")
    # sampled dL/dx parity for the same tokens
    xs = r(x[tok]).requires_grad_()
    oracle.experts_forward(xs, r(W1), r(W2), mask[:, tok], s[:, tok]).backward(r(dy[tok]))
    assert_close(xd.grad.reshape(M, D)[tok], xs.grad, "G_x (sampled tokens)")


def test_skewed_routing_with_shared_experts_full_size():
    # D=2048, H=1408, 60 routed + 4 shared experts, 4 routed + 4 shared per token, 16384 tokens,
    # Zipf-like load: a few experts hold ~10x the mean, the shared ones hold every token
    _sampled_parity_on_device_inputs(16384, 2048, 1408, 64, 8, 4, 1.8, 0, 8, experts=(0, 59))


def test_headline_layer_full_size_with_everything_saved():
    # the headline layer at save_percent=100: every row takes the saved-pre-activation branch
    # of the SwiGLU backward (momoe/momoe.py:486-491)
    _sampled_parity_on_device_inputs(8192, 2048, 1024, 128, 8, 0, None, 100, 4, experts=(0, 77, 127))


@pytest.mark.parametrize("sp", [0, 50, 100])
def test_memory_stress_layer_full_size(sp):
    # D=4096, H=2048, N=64, K=8, 65536 tokens: 524288 sorted rows, 4 GiB intermediates
    _sampled_parity_on_device_inputs(65536, 4096, 2048, 64, 8, 0, None, sp, 16, experts=(63,), n_tok=8)


def test_input_formats_and_partial_gradients():
    # what a caller may hand over besides the router's own outputs: fp32 x (cast to bf16 like
    # the reference, momoe/momoe.py:863), non-contiguous x and G_y, a contiguous s_NM, a strided
    # mask; and backward with only some inputs requiring gradients.
    import momoe_amd
    M, D, H, N, K = 384, 128, 96, 10, 3
    x, W1, W2, mask, s, dy = make_layer_inputs(M, D, H, N, K, seed=21)
    ref = run_oracle_layer(x, W1, W2, mask, s, dy)
    dev = "cuda:0"
    layer = momoe_amd.MoMoE(D, H, N, K, 0, Wl1_ND2H=W1.to(dev), Wl2_NHD=W2.to(dev))
    # the oracle sees bf16-rounded x: hand the device the same values as fp32, in a strided view
    x32 = x.to(torch.bfloat16).float()
    wide = torch.zeros(M, 2 * D, device=dev)
    wide[:, ::2] = x32.to(dev)
    xd = wide[:, ::2].reshape(2, M // 2, D).requires_grad_()
    assert not xd.is_contiguous() or xd.dtype == torch.float32
    sd = s.contiguous().to(dev).requires_grad_()                      # plain [N, M]
    maskd = mask.T.contiguous().to(dev).T                             # strides (1, N)
    y, sizes = layer(xd, maskd, sd)
    assert y.dtype == torch.bfloat16 and y.shape == (2, M // 2, D) and sizes.dtype == torch.int64
    dy_wide = torch.zeros(2, M // 2, 2 * D, device=dev, dtype=torch.bfloat16)
    dy_wide[..., ::2] = dy.to(dev, torch.bfloat16).reshape(2, M // 2, D)
    y.backward(dy_wide[..., ::2])
    torch.cuda.synchronize()
    assert torch.equal(sizes.cpu(), ref["sizes"])
    assert_close(y.reshape(M, D), ref["y"], "y")
    assert_close(xd.grad.reshape(M, D), ref["G_x"], "G_x")
    assert_close(sd.grad, ref["G_s"], "G_s")
    assert_close(layer.Wl1_ND2H.grad, ref["G_W1"], "G_W1")
    assert_close(layer.Wl2_NHD.grad, ref["G_W2"], "G_W2")

    # frozen experts: only x and s get gradients; then only the weights
    frozen = momoe_amd.MoMoE(D, H, N, K, 50, Wl1_ND2H=W1.to(dev), Wl2_NHD=W2.to(dev))
    for p in frozen.parameters():
        p.requires_grad_(False)
    xb = x.to(dev, torch.bfloat16).reshape(1, M, D).requires_grad_()
    sb = s.contiguous().to(dev).requires_grad_()
    yb, _ = frozen(xb, mask.to(dev), sb)
    yb.backward(dy.to(dev, torch.bfloat16).reshape(1, M, D))
    assert frozen.Wl1_ND2H.grad is None and frozen.Wl2_NHD.grad is None
    assert_close(xb.grad.reshape(M, D), ref["G_x"], "G_x (frozen experts)")
    assert_close(sb.grad, ref["G_s"], "G_s (frozen experts)")
    xc = x.to(dev, torch.bfloat16).reshape(1, M, D)
    yc, _ = layer(xc, mask.to(dev), s.contiguous().to(dev))
    layer.zero_grad(set_to_none=True)
    yc.backward(dy.to(dev, torch.bfloat16).reshape(1, M, D))
    assert_close(layer.Wl1_ND2H.grad, ref["G_W1"], "G_W1 (weights only)")
    assert_close(layer.Wl2_NHD.grad, ref["G_W2"], "G_W2 (weights only)")
    # no_grad forward keeps nothing for a backward
    with torch.no_grad():
        yn, _ = layer(xc, mask.to(dev), s.contiguous().to(dev))
    assert not yn.requires_grad and torch.equal(yn, yc.detach())


def test_recomputing_gemm_ignores_a_table_of_taller_tiles():
    """momoe_lin1_swiglu_bwd takes row tiles of at most 256 rows: given the 320-row table of the other
    GEMMs it must leave its outputs alone instead of computing on tiles it cannot hold."""
    from momoe_amd import _hip
    M, D, H, N, K = 2048, 128, 64, 2, 1
    x, W1, _, mask, s, _ = make_layer_inputs(M, D, H, N, K, seed=5)
    dev = "cuda:0"
    ib = _hip.index_build(mask.to(dev), K, tile_rows=_hip.TILE_ROWS)
    msum = M * K
    assert _hip.TILE_ROWS > _hip.RECOMPUTE_TILE_ROWS and int(ib["sizes_N"].max()) > _hip.RECOMPUTE_TILE_ROWS
    u = torch.randn(msum, H, device=dev).to(torch.bfloat16)
    xb, W1b, sd = x.to(dev).to(torch.bfloat16), W1.to(dev), s.to(dev)

    def run(table):
        gz = torch.full((2 * H // 32, msum, 32), 7.0, device=dev, dtype=torch.bfloat16)
        hsT = torch.full((_hip.padded_rows(msum, N) // 32, H, 32), 7.0, device=dev, dtype=torch.bfloat16)
        gs_part = torch.full(((H + _hip.GS_BLOCK - 1) // _hip.GS_BLOCK, msum), 7.0, device=dev)
        _hip.lin1_swiglu_bwd(xb, W1b, ib["idx_Msum"], table, u, sd, 0, gz, hsT, gs_part)
        torch.cuda.synchronize()
        return gz, hsT, gs_part

    for t in run(ib["tile_table"]):
        assert bool((t == 7.0).all())
    own = _hip.tile_table_build(ib["cumsums_N"], M, K, _hip.RECOMPUTE_TILE_ROWS)
    assert not bool((run(own)[0] == 7.0).all())


@pytest.mark.parametrize("sp", [0, 40])
def test_both_row_tile_geometries_give_the_same_layer(sp):
    """Experts of 1..700 rows on 256-row and on 320-row tiles (and on the library's own choice): the
    contraction order does not depend on the tile height, so every result is bit-identical, and
    the 320-row path is checked against the oracle like any other."""
    from momoe_amd import _hip, experts
    M, D, H, N, K = 1500, 160, 96, 12, 3
    x, W1, W2, mask, s, dy = make_layer_inputs(M, D, H, N, K, seed=21, skew=1.2)
    assert int(mask.sum(1).max()) > 2 * _hip.RECOMPUTE_TILE_ROWS  # several tiles, ragged
    outs = {}
    try:
        for rows in (_hip.RECOMPUTE_TILE_ROWS, _hip.TILE_ROWS, _hip.AUTO_TILE_ROWS, 288):
            experts.TILE_ROWS = rows
            outs[rows] = run_device_layer(x, W1, W2, mask, s, dy, K, sp)
    finally:
        experts.TILE_ROWS = _hip.AUTO_TILE_ROWS
    ref = run_oracle_layer(x, W1, W2, mask, s, dy)
    _check_all(outs[_hip.TILE_ROWS], ref)
    base = outs[_hip.RECOMPUTE_TILE_ROWS]
    for rows, got in outs.items():
        for k in base:
            assert torch.equal(got[k], base[k]), (rows, k)
