"""Seeded synthetic inputs shared by the CPU and GPU parity tests.

All tensors are generated on the CPU from one torch.Generator so the oracle and
the device path see identical bits.
"""
import torch


def make_routing(M, N, K, Ks=0, seed=0, skew=None):
    """fp32 N(0,1) logits -> (mask_NM int32 [N,M], s_NM fp32 [N,M] as a transposed view).

    Routed experts: top-(K-Ks) of the logits, weights = softmax over the selected
    logits.  Shared experts (the last Ks rows): all-ones mask rows, weights =
    softmax over the Ks shared logits.  `skew` adds a per-expert offset
    -skew*ln(rank) to the routed logits.
    """
    g = torch.Generator().manual_seed(seed)
    Ng = N - Ks
    logits = torch.randn(M, N, generator=g)
    if skew:
        logits[:, :Ng] += -skew * torch.log(torch.arange(1, Ng + 1, dtype=torch.float32))[None, :]
    p = torch.softmax(logits[:, :Ng], dim=-1)
    _, sel = torch.topk(p, K - Ks, dim=-1)
    selmask = torch.zeros(M, Ng, dtype=torch.bool).scatter_(1, sel, True)
    w = p * selmask
    s_MN = torch.cat([w / w.sum(-1, keepdim=True), torch.softmax(logits[:, Ng:], dim=-1)], dim=-1)
    mask_NM = torch.ones(N, M, dtype=torch.int32)
    mask_NM[:Ng] = selmask.T.to(torch.int32)
    return mask_NM.contiguous(), s_MN.contiguous().T


def make_layer_inputs(M, D, H, N, K, Ks=0, seed=0, skew=None, wstd=0.02):
    g = torch.Generator().manual_seed(seed + 1000)
    x = torch.randn(M, D, generator=g)
    W1 = torch.randn(N, D, 2 * H, generator=g) * wstd
    W2 = torch.randn(N, H, D, generator=g) * wstd
    dy = torch.randn(M, D, generator=g)
    mask, s = make_routing(M, N, K, Ks, seed=seed, skew=skew)
    return x, W1, W2, mask, s, dy
