"""Helpers for the GPU parity tests: run the HIP path and the CPU oracle on the same bits."""
import torch

import oracle

RTOL = 2e-2  # tolerance stated for bf16 results against the fp32-accumulated oracle
ATOL = 2e-2


def rel_err(got, ref):
    got, ref = got.detach().float().cpu(), ref.detach().float().cpu()
    return ((got - ref).norm() / ref.norm().clamp_min(1e-30)).item()


# Size of the error the cap on plain-check misses is computed for, relative to the RMS of the
# reference: half of the norm-wise bound the same check enforces (relative L2 error < 1e-2), and
# about twice what is measured (1.5e-3 .. 3e-3).
MODEL_REL_ERR = 5e-3


def _scale_of(ref):
    if ref.dim() == 3:  # per-expert weight gradients: each expert has its own scale
        return ref.pow(2).mean(dim=(1, 2), keepdim=True).sqrt()
    return ref.pow(2).mean().sqrt().reshape(())


def plain_miss_cap(ref):
    """How many elements may miss the PLAIN rtol/atol 2e-2 check: the number a Gaussian error of
    standard deviation MODEL_REL_ERR * rms(ref) (per expert for weight gradients) would leave
    outside it, plus four standard deviations of that count and 2."""
    ref = ref.detach().double().cpu()
    sigma = (MODEL_REL_ERR * _scale_of(ref)).clamp_min(1e-30)
    expected = torch.erfc((ATOL + RTOL * ref.abs()) / (sigma * 2 ** 0.5)).sum().item()
    return int(expected + 4 * expected ** 0.5 + 2)


def tolerance_report(got, ref):
    """(elements outside the plain rtol/atol 2e-2 check, elements outside the check whose
    absolute term is scaled by max(1, rms(ref)), the scale used, relative L2 error)."""
    got, ref = got.detach().float().cpu(), ref.detach().float().cpu()
    scale = _scale_of(ref).clamp_min(1.0)
    if ref.dim() != 3:
        scale = scale.item()
    diff = (got - ref).abs()
    plain = int((diff > ATOL + RTOL * ref.abs()).sum())
    scaled = int((diff > ATOL * scale + RTOL * ref.abs()).sum())
    return plain, scaled, scale, rel_err(got, ref)


def assert_close(got, ref, what, rel=1e-2):
    """Elementwise |got-ref| <= ATOL*max(1, rms(ref)) + RTOL*|ref|, a norm-wise bound, and a cap
    on the number of elements outside the plain rtol/atol 2e-2 check.

    For tensors whose RMS is at most 1 (y, G_x, and the weight gradients of small experts)
    this is the plain rtol/atol 2e-2 check.  The absolute term follows the RMS of larger
    tensors (per expert for the weight gradients, and dL/ds): the operands of the GEMMs behind
    them (G_z, h, the scaled G_y) are bf16 in the reference too (momoe/momoe.py:340, 533-535,
    555, and dL/ds is formed from the bf16 h or the bf16 y_pre, :685-697), their rounding
    accumulates over the contraction and scales with the result itself, so the reference's own
    arithmetic misses the plain check on those tensors by the same margin
    (tests/test_oracle_experts.py::test_reference_rounding_alone_breaks_the_plain_tolerance).
    How many elements may miss the plain check is capped (`plain_miss_cap`), so the relaxation
    cannot drift; whenever it matters the count and the cap are printed (pytest -rP / -s).
    """
    got, ref = got.detach().float().cpu(), ref.detach().float().cpu()
    plain, scaled, _, e = tolerance_report(got, ref)
    cap = plain_miss_cap(ref) if plain else 0
    if plain:
        print(f"[tolerance] {what}: {plain}/{ref.numel()} elements outside plain rtol/atol 2e-2 "
              f"(cap {cap}), {scaled} outside the RMS-scaled check; rms(ref) "
              f"{ref.pow(2).mean().sqrt().item():.3g}, relative L2 error {e:.2e}")
    assert scaled == 0, (f"{what}: {scaled}/{ref.numel()} elements outside tolerance, "
                         f"max abs diff {(got - ref).abs().max().item():.4g}, rms(ref) "
                         f"{ref.pow(2).mean().sqrt().item():.4g}, relative L2 error {e:.3e}")
    assert plain <= cap, (f"{what}: {plain}/{ref.numel()} elements outside the plain rtol/atol 2e-2 "
                          f"check, more than the {cap} an error of {MODEL_REL_ERR:g} x rms(ref) "
                          f"= {MODEL_REL_ERR * ref.pow(2).mean().sqrt().item():.3g} explains")
    assert e < rel, f"{what}: relative L2 error {e:.3e} >= {rel}"


def run_device_layer(x, W1, W2, mask, s, dy, K, save_percent, B=1):
    """Forward+backward of momoe_amd.MoMoE on cuda:0; returns CPU tensors."""
    import momoe_amd

    dev = "cuda:0"
    M, D = x.shape
    N, H = W2.shape[0], W2.shape[1]
    layer = momoe_amd.MoMoE(D, H, N, K, save_percent=save_percent, Wl1_ND2H=W1.to(dev), Wl2_NHD=W2.to(dev))
    xd = x.to(dev, torch.bfloat16).reshape(B, M // B, D).requires_grad_()
    sd = s.T.contiguous().to(dev).T.requires_grad_()  # transposed view, like the router's output
    y, sizes = layer(xd, mask.to(dev), sd)
    y.backward(dy.to(dev, torch.bfloat16).reshape(B, M // B, D))
    torch.cuda.synchronize()
    return {
        "y": y.detach().reshape(M, D).cpu(), "sizes": sizes.cpu(),
        "G_x": xd.grad.reshape(M, D).cpu(), "G_W1": layer.Wl1_ND2H.grad.cpu(),
        "G_W2": layer.Wl2_NHD.grad.cpu(), "G_s": sd.grad.cpu(),
    }


def run_oracle_layer(x, W1, W2, mask, s, dy, dtype=torch.float32):
    """Oracle on the bf16-rounded inputs the device sees, arithmetic in `dtype`."""
    r = lambda t: t.to(torch.bfloat16).to(dtype)
    xo = r(x).requires_grad_()
    W1o = r(W1).requires_grad_()
    W2o = r(W2).requires_grad_()
    so = s.to(dtype).clone().requires_grad_()
    y = oracle.experts_forward(xo, W1o, W2o, mask, so, dtype=dtype)
    y.backward(r(dy))
    return {"y": y.detach(), "G_x": xo.grad, "G_W1": W1o.grad, "G_W2": W2o.grad, "G_s": so.grad,
            "sizes": (mask != 0).sum(1).to(torch.int64)}


def device_layer_inputs(M, D, H, N, K, Ks=0, skew=None, seed=77, routing_seed=3):
    """x, dy, Wl1, Wl2 drawn on the GPU in bf16 (the host would take minutes at the full
    sizes) plus CPU routing (mask_NM, s_NM) from `helpers.make_routing`."""
    from helpers import make_routing
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(seed)
    x = torch.randn(M, D, generator=g, device=dev).to(torch.bfloat16)
    dy = torch.randn(M, D, generator=g, device=dev).to(torch.bfloat16)
    W1 = torch.empty(N, D, 2 * H, device=dev, dtype=torch.bfloat16).normal_(0, 0.02, generator=g)
    W2 = torch.empty(N, H, D, device=dev, dtype=torch.bfloat16).normal_(0, 0.02, generator=g)
    mask, s = make_routing(M, N, K, Ks, seed=routing_seed, skew=skew)
    return x, dy, W1, W2, mask, s


def oracle_forward_for_tokens(x, W1, W2, mask, s, tok):
    """Oracle forward for the tokens `tok` (CPU index tensor) of device-resident x / weights,
    restricted to the experts those tokens use.  Returns (y fp32 [len(tok), D], the fp32 copy
    of x[tok] with requires_grad set, so the caller can continue into the backward)."""
    f = lambda t: t.detach().float().cpu()
    dev = x.device
    used = torch.nonzero(mask[:, tok].sum(1)).flatten()
    xs = f(x[tok.to(dev)]).requires_grad_()
    yo = oracle.experts_forward(xs, f(W1[used.to(dev)]), f(W2[used.to(dev)]), mask[used][:, tok],
                                s[used][:, tok])
    return yo, xs


def sampled_parity_on_device_inputs(M, D, H, N, K, Ks, skew, sp, B, experts, n_tok=16):
    """Full-size layer forward + backward; the oracle sees the same bits, copied back for a
    sample of tokens and experts only."""
    import momoe_amd
    dev = "cuda:0"
    x, dy, W1, W2, mask, s = device_layer_inputs(M, D, H, N, K, Ks, skew)
    layer = momoe_amd.MoMoE(D, H, N, K, sp, Wl1_ND2H=W1, Wl2_NHD=W2)
    xd = x.reshape(B, M // B, D).clone().requires_grad_()
    sd = s.T.contiguous().to(dev).T.requires_grad_()
    y, sizes = layer(xd, mask.to(dev), sd)
    y.backward(dy.reshape(B, M // B, D))
    torch.cuda.synchronize()
    assert torch.equal(sizes.cpu(), (mask != 0).sum(1))
    assert torch.isfinite(y).all() and torch.isfinite(xd.grad).all()
    assert torch.isfinite(layer.Wl1_ND2H.grad).all() and torch.isfinite(layer.Wl2_NHD.grad).all()
    f = lambda t: t.detach().float().cpu()
    # sampled tokens: forward and dL/dx against the oracle restricted to the experts they use
    tok = torch.arange(0, M, M // n_tok)[:n_tok]
    yo, xs = oracle_forward_for_tokens(x, W1, W2, mask, s, tok)
    assert_close(y.reshape(M, D)[tok.to(dev)], yo, "y (sampled tokens)")
    yo.backward(f(dy[tok.to(dev)]))
    assert_close(xd.grad.reshape(M, D)[tok.to(dev)], xs.grad, "G_x (sampled tokens)")
    # sampled experts: weight gradients and dL/ds from the closed form
    for i in experts:
        sel = torch.nonzero(mask[i]).flatten()
        one = torch.ones(1, sel.numel(), dtype=torch.int32)
        _, gW1, gW2, gs = oracle.experts_backward_closed_form(
            f(x[sel.to(dev)]), f(W1[i:i + 1]), f(W2[i:i + 1]), one, s[i:i + 1, sel], f(dy[sel.to(dev)]),
            dtype=torch.float32)
        assert_close(layer.Wl1_ND2H.grad[i], gW1[0], f"G_W1[{i}]")
        assert_close(layer.Wl2_NHD.grad[i], gW2[0], f"G_W2[{i}]")
        assert_close(sd.grad[i, sel.to(dev)], gs[0], f"G_s[{i}]")
