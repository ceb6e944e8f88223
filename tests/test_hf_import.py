"""Packing of Hugging Face style expert weights into the MoMoE layout.

The reference of these tests is the published Qwen3-MoE block written out with
torch.nn.functional (softmax over all experts, top-k, renormalise, per expert
down_proj(silu(gate_proj(x)) * up_proj(x))); the packed weights go through the oracle
(CPU) and through the HIP modules (GPU)."""
import json
import os

import pytest
import torch
import torch.nn.functional as F

import oracle
from momoe_amd import hf_import


def _hf_block(x, gate_w, experts, k):
    """x [M,D]; gate_w [N,D]; experts: list of (gate_proj [H,D], up_proj [H,D], down_proj [D,H])."""
    logits = F.linear(x, gate_w)
    p = torch.softmax(logits.float(), dim=-1)
    w, sel = torch.topk(p, k, dim=-1)
    w = w / w.sum(-1, keepdim=True)
    y = torch.zeros_like(x)
    for m in range(x.shape[0]):
        for j in range(k):
            g, u, d = experts[int(sel[m, j])]
            y[m] += w[m, j] * F.linear(F.silu(F.linear(x[m], g)) * F.linear(x[m], u), d)
    return y, sel, w


def _random_checkpoint(N, D, H, layer, seed=0):
    g = torch.Generator().manual_seed(seed)
    t = {f"model.layers.{layer}.mlp.gate.weight": torch.randn(N, D, generator=g) * 0.5}
    for e in range(N):
        p = f"model.layers.{layer}.mlp.experts.{e}."
        t[p + "gate_proj.weight"] = torch.randn(H, D, generator=g) * 0.2
        t[p + "up_proj.weight"] = torch.randn(H, D, generator=g) * 0.2
        t[p + "down_proj.weight"] = torch.randn(D, H, generator=g) * 0.2
    t["model.layers.%d.self_attn.q_proj.weight" % layer] = torch.zeros(4, 4)
    return t


def _experts_of(t, layer, N):
    p = f"model.layers.{layer}.mlp.experts."
    return [(t[f"{p}{e}.gate_proj.weight"], t[f"{p}{e}.up_proj.weight"], t[f"{p}{e}.down_proj.weight"])
            for e in range(N)]


def test_packed_weights_reproduce_the_hf_block_through_the_oracle():
    N, D, H, K, M, layer = 6, 16, 24, 2, 40, 3
    t = _random_checkpoint(N, D, H, layer)
    w = hf_import.qwen3_moe_layer_tensors(t, layer, dtype=torch.float32)
    assert (w["N"], w["D"], w["H"]) == (N, D, H)
    assert w["Wl1_ND2H"].shape == (N, D, 2 * H) and w["Wl2_NHD"].shape == (N, H, D)
    assert w["Wl1_ND2H"].is_contiguous() and w["Wl2_NHD"].is_contiguous() and w["Wg_DN"].is_contiguous()
    x = torch.randn(M, D, generator=torch.Generator().manual_seed(1))
    want, sel, wts = _hf_block(x, t[f"model.layers.{layer}.mlp.gate.weight"], _experts_of(t, layer, N), K)
    # fp32 logits (the oracle's own gate matmul rounds through bf16 as the reference does)
    r = oracle.router_forward(None, None, torch.zeros(N), N, K, 0, logits=x @ w["Wg_DN"])
    assert torch.equal(r["mask_NM"].T.bool(), torch.zeros(M, N, dtype=torch.bool).scatter_(1, sel, True))
    got = oracle.experts_forward(x, w["Wl1_ND2H"], w["Wl2_NHD"], r["mask_NM"], r["s_NM"])
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-6)
    # swapping the halves is the mistake this guards against: it must not pass
    swapped = torch.cat([w["Wl1_ND2H"][:, :, H:], w["Wl1_ND2H"][:, :, :H]], dim=-1)
    bad = oracle.experts_forward(x, swapped, w["Wl2_NHD"], r["mask_NM"], r["s_NM"])
    assert (bad - want).abs().max() > 1e-3


def test_pack_unpack_round_trip_and_shape_errors():
    g = torch.Generator().manual_seed(2)
    gate, up, down = torch.randn(3, 8, 4, generator=g), torch.randn(3, 8, 4, generator=g), torch.randn(3, 4, 8, generator=g)
    Wl1, Wl2 = hf_import.pack_experts(gate, up, down, dtype=torch.float32)
    g2, u2, d2 = hf_import.unpack_experts(Wl1, Wl2)
    assert torch.equal(g2, gate) and torch.equal(u2, up) and torch.equal(d2, down)
    assert hf_import.pack_experts(list(gate), list(up), list(down))[0].dtype == torch.bfloat16
    with pytest.raises(ValueError):
        hf_import.pack_experts(gate, up, down.transpose(1, 2))
    with pytest.raises(ValueError):
        hf_import.pack_experts(gate, up[:, :4], down)
    with pytest.raises(KeyError):
        hf_import.qwen3_moe_layer_tensors({}, 0)
    t = _random_checkpoint(2, 4, 8, 0)
    del t["model.layers.0.mlp.experts.1.down_proj.weight"]
    with pytest.raises(KeyError):
        hf_import.qwen3_moe_layer_tensors(t, 0)


def test_sharded_safetensors_directory(tmp_path):
    from safetensors.torch import save_file
    N, D, H, layer = 4, 8, 16, 1
    t = _random_checkpoint(N, D, H, layer)
    names = sorted(t)
    shards = {"model-00001-of-00002.safetensors": names[::2], "model-00002-of-00002.safetensors": names[1::2]}
    weight_map = {}
    for fname, keys in shards.items():
        save_file({k: t[k].contiguous() for k in keys}, os.path.join(tmp_path, fname))
        weight_map.update({k: fname for k in keys})
    want = hf_import.qwen3_moe_layer_tensors(t, layer)
    # without an index the files are scanned; with one it is trusted
    for with_index in (False, True):
        if with_index:
            with open(os.path.join(tmp_path, "model.safetensors.index.json"), "w") as f:
                json.dump({"metadata": {}, "weight_map": weight_map}, f)
        got = hf_import.load_qwen3_moe_layer(str(tmp_path), layer)
        for k in ("Wg_DN", "Wl1_ND2H", "Wl2_NHD"):
            assert got[k].dtype == torch.bfloat16 and torch.equal(got[k], want[k])
    with pytest.raises(FileNotFoundError):
        hf_import.SafetensorsDir(str(tmp_path / "nothing"))


@pytest.mark.gpu
def test_moe_built_from_checkpoint_matches_the_hf_block_on_device():
    N, D, H, K, M, layer = 8, 64, 96, 2, 96, 5
    t = {k: v.to(torch.bfloat16).float() for k, v in _random_checkpoint(N, D, H, layer, seed=3).items()}
    # small gate logits: the router rounds them to bf16 (momoe/topk_router.py:92-95), and the
    # rounding of a logit of size 4 would move a gate weight by more than the tolerance
    rk = f"model.layers.{layer}.mlp.gate.weight"
    t[rk] = (t[rk] * 0.1).to(torch.bfloat16).float()
    moe = hf_import.moe_from_qwen3(t, layer, K)
    x = torch.randn(M, D, generator=torch.Generator().manual_seed(4)).to(torch.bfloat16)
    y = moe(x.view(2, M // 2, D).cuda()).float().cpu().view(M, D)
    want, _, _ = _hf_block(x.float(), t[rk], _experts_of(t, layer, N), K)
    # tokens whose k-th and (k+1)-th probabilities are within bf16 rounding may route differently
    p = torch.softmax(F.linear(x.float(), t[rk]), -1)
    top = torch.topk(p, K + 1, dim=-1).values
    clear = (top[:, K - 1] - top[:, K]) > 1e-2 * top[:, K - 1]
    assert clear.float().mean() > 0.7
    from gpu_util import assert_close
    assert_close(y[clear], want[clear], "y of the packed Qwen3-style block")
    assert torch.all(moe.biases_N == 0)  # selection bias stays frozen
