"""Helpers for the GPU parity tests: run the HIP path and the CPU oracle on the same bits."""
import torch

import oracle

RTOL = 2e-2  # tolerance stated for bf16 results against the fp32-accumulated oracle
ATOL = 2e-2


def rel_err(got, ref):
    got, ref = got.detach().float().cpu(), ref.detach().float().cpu()
    return ((got - ref).norm() / ref.norm().clamp_min(1e-30)).item()


def assert_close(got, ref, what, rel=1e-2):
    """Elementwise |got-ref| <= ATOL*max(1, rms(ref)) + RTOL*|ref| and a norm-wise bound.

    For tensors whose RMS is at most 1 (y, G_x, G_s and the weight gradients of small
    experts) this is the plain rtol/atol 2e-2 check.  The absolute term follows the RMS
    of larger tensors (per expert for the weight gradients) because the bf16 rounding of the MFMA inputs of the weight-gradient
    GEMMs (G_z and h are bf16 in the reference too, momoe/momoe.py:555-556) accumulates
    over the contraction and scales with the result itself.
    """
    got, ref = got.detach().float().cpu(), ref.detach().float().cpu()
    e = rel_err(got, ref)
    if ref.dim() == 3:  # per-expert weight gradients: each expert has its own scale
        scale = ref.pow(2).mean(dim=(1, 2), keepdim=True).sqrt().clamp_min(1.0)
    else:
        scale = max(1.0, ref.pow(2).mean().sqrt().item())
    bad = (got - ref).abs() > ATOL * scale + RTOL * ref.abs()
    assert not bad.any(), (f"{what}: {int(bad.sum())}/{bad.numel()} elements outside tolerance, "
                           f"max abs diff {(got - ref).abs().max().item():.4g}, rms(ref) "
                           f"{ref.pow(2).mean().sqrt().item():.4g}, relative L2 error {e:.3e}")
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
