"""The hand-worked vectors of tests/golden/hand_cases.json (plain Python arithmetic, see
make_hand_cases.py) against the oracle (CPU) and against the HIP path (GPU)."""
import json
import os

import numpy as np
import pytest
import torch

import oracle

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hand_cases.json")) as f:
    CASES = json.load(f)


def test_oracle_index_matches_hand_case():
    c = CASES["index"]
    out = oracle.index_build(np.array(c["mask_NM"], dtype=np.int32))
    for k in ("sizes_N", "cumsums_N", "idx_Msum", "which_Msum"):
        assert out[k].tolist() == c[k], k
    assert out["inv_MK"].tolist() == c["inv_MK"]


def _experts_inputs(c, key):
    t = lambda v, dt=torch.float32: torch.tensor(v, dtype=dt)
    return t(c[key]), t(c["Wl1_ND2H"]), t(c["Wl2_NHD"]), t(c["mask_NM"], torch.int32), t(c["s_NM"])


@pytest.mark.parametrize("key", ["x", "x_zero_gate"])
def test_oracle_experts_match_hand_case(key):
    c = CASES["experts"]
    y = oracle.experts_forward(*_experts_inputs(c, key))
    torch.testing.assert_close(y, torch.tensor(c["y" + key[1:]]), rtol=1e-6, atol=1e-7)


def test_oracle_router_matches_hand_case():
    c = CASES["router"]
    lg = torch.tensor(c["logits_MN"])
    out = oracle.router_forward(None, None, torch.zeros(4), 4, c["K"], c["Ks"], logits=lg)
    assert out["mask_NM"].T.tolist() == c["mask_MN"]
    torch.testing.assert_close(out["s_NM"].T, torch.tensor(c["s_MN"]), rtol=1e-6, atol=1e-7)


@pytest.mark.gpu
def test_device_index_matches_hand_case():
    from momoe_amd import _hip
    c = CASES["index"]
    ib = _hip.index_build(torch.tensor(c["mask_NM"], dtype=torch.int32, device="cuda:0"), c["K"])
    torch.cuda.synchronize()
    assert ib["sizes_N"].tolist() == c["sizes_N"] and ib["cumsums_N"].tolist() == c["cumsums_N"]
    assert ib["idx_Msum"].tolist() == c["idx_Msum"] and ib["which_Msum"].tolist() == c["which_Msum"]
    assert ib["inv_MK"].tolist() == c["inv_MK"] and ib["violations"].item() == 0


@pytest.mark.gpu
def test_device_experts_match_hand_case():
    # the kernels need D and H to be multiples of 32: the 2x1 case is embedded in zero padding
    import momoe_amd
    c = CASES["experts"]
    x, W1, W2, mask, s = _experts_inputs(c, "x")
    D, H, N = 32, 32, 2
    W1p = torch.zeros(N, D, 2 * H)
    W1p[:, :2, 0] = W1[:, :, 0]   # linear half: first H columns
    W1p[:, :2, H] = W1[:, :, 1]   # SiLU half: last H columns
    W2p = torch.zeros(N, H, D)
    W2p[:, 0, :2] = W2[:, 0, :]
    xp = torch.zeros(2, D)
    xp[:, :2] = x
    layer = momoe_amd.MoMoE(D, H, N, 1, 0, Wl1_ND2H=W1p.to("cuda:0"), Wl2_NHD=W2p.to("cuda:0"))
    y, sizes = layer(xp.to("cuda:0").reshape(1, 2, D), mask.to("cuda:0"), s.to("cuda:0"))
    assert sizes.tolist() == [1, 1]
    # every input is exactly representable in bf16; the outputs are rounded to bf16
    torch.testing.assert_close(y.float().cpu().reshape(2, D)[:, :2], torch.tensor(c["y"]), rtol=1e-2, atol=1e-3)
    assert torch.all(y.reshape(2, D)[:, 2:] == 0)


@pytest.mark.gpu
def test_device_router_matches_hand_case():
    from momoe_amd import _hip
    c = CASES["router"]
    lg = torch.tensor(c["logits_MN"], device="cuda:0")
    mask, s_MN, _, _, _ = _hip.router_fwd(lg, torch.zeros(4, device="cuda:0"), c["K"], c["Ks"])
    assert mask.T.tolist() == c["mask_MN"]
    torch.testing.assert_close(s_MN.cpu(), torch.tensor(c["s_MN"]), rtol=1e-5, atol=1e-7)
