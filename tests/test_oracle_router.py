"""Pins the router oracle: library special case, brute-force top-k, autograd
through an independent differentiable restatement, and the bias rule."""
import pytest
import torch

import oracle


def _logits(M, N, seed):
    return torch.randn(M, N, generator=torch.Generator().manual_seed(seed))


def test_no_shared_no_bias_is_softmax_over_topk_logits():
    M, N, K = 50, 16, 4
    lg = _logits(M, N, 0)
    r = oracle.router_forward(None, None, torch.zeros(N), N, K, 0, logits=lg)
    vals, sel = torch.topk(lg, K, dim=-1)
    ref = torch.zeros(M, N).scatter_(1, sel, torch.softmax(vals, dim=-1))
    torch.testing.assert_close(r["s_NM"].T, ref, rtol=1e-5, atol=1e-6)
    refmask = torch.zeros(M, N, dtype=torch.int32).scatter_(1, sel, 1)
    assert torch.equal(r["mask_NM"], refmask.T)
    assert r["mask_NM"].dtype == torch.int32
    assert r["s_NM"].stride() == (1, N)  # transposed view of an [M,N] matrix


def test_bias_moves_selection_but_not_weights():
    M, N, K = 64, 8, 2
    lg = _logits(M, N, 1)
    bias = torch.zeros(N)
    bias[5] = 10.0  # expert 5 always selected
    r = oracle.router_forward(None, None, bias, N, K, 0, logits=lg)
    assert torch.all(r["mask_NM"][5] == 1)
    # weights are still softmax over the selected logits (bias is not in s)
    m = r["mask_NM"].T.bool()
    ref = torch.softmax(lg.masked_fill(~m, float("-inf")), dim=-1)
    torch.testing.assert_close(r["s_NM"].T, ref, rtol=1e-5, atol=1e-6)


def test_bruteforce_topk_and_shared_group():
    M, N, K, Ks = 20, 10, 5, 2
    lg = _logits(M, N, 2)
    bias = torch.cat([torch.randn(N - Ks, generator=torch.Generator().manual_seed(9)) * 0.05,
                      torch.full((Ks,), float("-inf"))])
    r = oracle.router_forward(None, None, bias, N, K, Ks, logits=lg)
    Ng = N - Ks
    for m in range(M):
        p = torch.softmax(lg[m, :Ng], 0)
        order = sorted(range(Ng), key=lambda j: -(p[j] + bias[j]).item())[: K - Ks]
        assert sorted(torch.nonzero(r["mask_NM"][:Ng, m]).flatten().tolist()) == sorted(order)
        tot = sum(p[j] for j in order)
        for j in order:
            assert abs(r["s_NM"][j, m] - p[j] / tot) < 1e-6
        ps = torch.softmax(lg[m, Ng:], 0)
        torch.testing.assert_close(r["s_NM"][Ng:, m], ps, rtol=1e-5, atol=1e-6)
    assert torch.all(r["mask_NM"][Ng:] == 1)
    torch.testing.assert_close(r["s_NM"][:Ng].sum(0), torch.ones(M), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("Ks", [0, 3])
def test_backward_closed_form_matches_autograd(Ks):
    M, N, K = 30, 12, 5
    lg = _logits(M, N, 3).double()
    bias = torch.cat([torch.zeros(N - Ks), torch.full((Ks,), float("-inf"))])
    r = oracle.router_forward(None, None, bias, N, K, Ks, logits=lg.float())
    G_s = torch.randn(N, M, dtype=torch.float64, generator=torch.Generator().manual_seed(4))
    G_s = G_s * (r["mask_NM"] != 0)  # the experts' backward gives zeros off-mask
    lgr = lg.clone().requires_grad_()
    s = oracle.router_probs_differentiable(lgr, r["mask_NM"], Ks)
    torch.testing.assert_close(s.float(), r["s_NM"], rtol=1e-5, atol=1e-6)
    (s * G_s).sum().backward()
    # recompute the saved quantities in fp64 for a tight comparison
    Ng = N - Ks
    sel = (r["mask_NM"][:Ng].T != 0).double()
    p_g = torch.softmax(lg[:, :Ng], -1) * sel
    p_s = torch.softmax(lg[:, Ng:], -1)
    got = oracle.router_backward_closed_form(G_s, torch.cat([p_g, p_s], -1), s.detach(),
                                             p_g.sum(-1), p_s.sum(-1), r["mask_NM"], Ks)
    torch.testing.assert_close(got, lgr.grad, rtol=1e-9, atol=1e-11)
    # unselected routed experts receive exactly zero logit gradient
    assert torch.all(got[:, :Ng][sel == 0] == 0)


def test_bias_update_rule():
    b = torch.tensor([0.0, 0.0, 0.0, float("-inf")])
    sizes = torch.tensor([10, 2, 6, 12])
    out = oracle.bias_update(b, sizes, M=12, K=2, Ks=1, rate=0.5)  # c_avg = 12*1/3 = 4
    assert out[:3].tolist() == [-0.5, 0.5, -0.5] and out[3] == float("-inf")
    out = oracle.bias_update(torch.zeros(2), torch.tensor([3, 3]), M=6, K=1, Ks=0, rate=1.0)
    assert out.tolist() == [0.0, 0.0]  # sign(0) = 0


def test_moe_wrapper_runs_and_updates_bias():
    torch.manual_seed(0)
    D, H, N, K, Ks = 16, 8, 6, 3, 1
    moe = oracle.OracleMoE(D, H, N, K, Ks, bias_update_rate=1e-2,
                           Wg_DN=torch.randn(D, N), Wl1_ND2H=torch.randn(N, D, 2 * H) * 0.1,
                           Wl2_NHD=torch.randn(N, H, D) * 0.1)
    x = torch.randn(2, 10, D, requires_grad=True)
    y = moe(x)
    y.float().pow(2).mean().backward()
    assert y.shape == x.shape and x.grad is not None and moe.router.Wg_DN.grad is not None
    assert moe.biases_N[-1] == float("-inf")
    assert set(moe.state_dict().keys()) == {"biases_N", "router.Wg_DN", "momoe.Wl1_ND2H", "momoe.Wl2_NHD"}
