"""Packing of Hugging Face style SwiGLU expert weights into the MoMoE parameter layout.

An HF expert MLP computes `down_proj(silu(gate_proj(x)) * up_proj(x))` with `nn.Linear`
weights stored [out_features, in_features].  MoMoE computes `h = a * silu(b)` with
`a = x @ Wl1[i][:, :H]` (linear half) and `b = x @ Wl1[i][:, H:]` (SiLU half)
(momoe/momoe.py:111-113, 148), then `h @ Wl2[i]`.  Hence

    Wl1_ND2H[i, :, :H] = up_proj.weight.T      Wl1_ND2H[i, :, H:] = gate_proj.weight.T
    Wl2_NHD[i]         = down_proj.weight.T    Wg_DN = router gate.weight.T

The Qwen3-MoE block (the model family the reference acknowledges, README.md:62) routes with
softmax over all experts, top-k, renormalised over the chosen k: TopKRouter with no shared
experts and zero selection bias.

Only local data is read: a mapping name -> tensor, or a directory of `.safetensors` files
(opened with the safetensors reader, which executes nothing from the file).  Everything here
is tensor bookkeeping on whatever device the inputs live on; the modules built from the result
run on the GPU.
"""
import json
import os

import torch

_EXPERT_KEY = "{prefix}.{layer}.mlp.experts.{expert}.{proj}.weight"
_ROUTER_KEY = "{prefix}.{layer}.mlp.gate.weight"


def pack_experts(gate_proj, up_proj, down_proj, dtype=torch.bfloat16):
    """gate_proj, up_proj: N tensors [H, D] (or one [N, H, D]); down_proj: N tensors [D, H]
    (or one [N, D, H]).  Returns (Wl1_ND2H, Wl2_NHD), contiguous, in `dtype`."""
    gate = _stack(gate_proj)
    up = _stack(up_proj)
    down = _stack(down_proj)
    if gate.dim() != 3 or gate.shape != up.shape:
        raise ValueError(f"gate_proj {tuple(gate.shape)} and up_proj {tuple(up.shape)} must both be [N, H, D]")
    N, H, D = gate.shape
    if tuple(down.shape) != (N, D, H):
        raise ValueError(f"down_proj must be [N, D, H] = {(N, D, H)}, got {tuple(down.shape)}")
    Wl1 = torch.empty((N, D, 2 * H), dtype=dtype, device=gate.device)
    Wl1[:, :, :H] = up.transpose(1, 2)
    Wl1[:, :, H:] = gate.transpose(1, 2)
    Wl2 = down.transpose(1, 2).to(dtype).contiguous()
    return Wl1, Wl2


def unpack_experts(Wl1_ND2H, Wl2_NHD):
    """Inverse of pack_experts: (gate_proj [N,H,D], up_proj [N,H,D], down_proj [N,D,H])."""
    H = Wl1_ND2H.shape[2] // 2
    up = Wl1_ND2H[:, :, :H].transpose(1, 2).contiguous()
    gate = Wl1_ND2H[:, :, H:].transpose(1, 2).contiguous()
    return gate, up, Wl2_NHD.transpose(1, 2).contiguous()


def qwen3_moe_layer_tensors(tensors, layer, prefix="model.layers", dtype=torch.bfloat16):
    """Collect one decoder layer's sparse MoE block from a mapping name -> tensor with the
    Hugging Face Qwen3-MoE names (`<prefix>.<layer>.mlp.experts.<e>.{gate,up,down}_proj.weight`,
    `<prefix>.<layer>.mlp.gate.weight`).  `tensors` only needs `__contains__` and
    `__getitem__`.  Returns dict(Wg_DN, Wl1_ND2H, Wl2_NHD, N, D, H)."""
    def key(expert, proj):
        return _EXPERT_KEY.format(prefix=prefix, layer=layer, expert=expert, proj=proj)

    N = 0
    while key(N, "gate_proj") in tensors:
        N += 1
    if N == 0:
        raise KeyError(f"no expert weights named {key(0, 'gate_proj')}")
    for e in range(N):
        for proj in ("up_proj", "down_proj"):
            if key(e, proj) not in tensors:
                raise KeyError(f"missing {key(e, proj)}")
    Wl1, Wl2 = pack_experts([tensors[key(e, "gate_proj")] for e in range(N)],
                            [tensors[key(e, "up_proj")] for e in range(N)],
                            [tensors[key(e, "down_proj")] for e in range(N)], dtype=dtype)
    out = {"Wl1_ND2H": Wl1, "Wl2_NHD": Wl2, "N": N, "D": Wl1.shape[1], "H": Wl2.shape[1], "Wg_DN": None}
    rk = _ROUTER_KEY.format(prefix=prefix, layer=layer)
    if rk in tensors:
        Wg = tensors[rk]
        if tuple(Wg.shape) != (N, out["D"]):
            raise ValueError(f"{rk} must be [N, D] = {(N, out['D'])}, got {tuple(Wg.shape)}")
        out["Wg_DN"] = Wg.T.to(dtype).contiguous()
    return out


class SafetensorsDir:
    """Read-only name -> tensor view of a local checkpoint directory: one or more
    `.safetensors` files, with `model.safetensors.index.json` if the checkpoint is sharded.
    Tensors are read one at a time, so a whole model is never resident."""

    def __init__(self, path):
        from safetensors import safe_open
        self._open = safe_open
        self.path = path
        index = os.path.join(path, "model.safetensors.index.json")
        self._where = {}
        if os.path.exists(index):
            with open(index) as f:
                self._where = dict(json.load(f)["weight_map"])
        else:
            for name in sorted(os.listdir(path)):
                if name.endswith(".safetensors"):
                    with safe_open(os.path.join(path, name), framework="pt") as f:
                        for k in f.keys():
                            self._where[k] = name
        if not self._where:
            raise FileNotFoundError(f"no .safetensors files in {path}")

    def __contains__(self, key):
        return key in self._where

    def __getitem__(self, key):
        with self._open(os.path.join(self.path, self._where[key]), framework="pt") as f:
            return f.get_tensor(key)


def load_qwen3_moe_layer(checkpoint_dir, layer, prefix="model.layers", dtype=torch.bfloat16):
    """qwen3_moe_layer_tensors over a local checkpoint directory."""
    return qwen3_moe_layer_tensors(SafetensorsDir(checkpoint_dir), layer, prefix=prefix, dtype=dtype)


def moe_from_qwen3(tensors, layer, num_experts_per_tok, save_percent=0, prefix="model.layers",
                   device="cuda"):
    """Build a `MoE` (router + experts, no shared experts, selection bias frozen at zero) from
    one layer of a Qwen3-MoE style checkpoint (a mapping or a SafetensorsDir)."""
    from .moe import MoE
    w = qwen3_moe_layer_tensors(tensors, layer, prefix=prefix)
    if w["Wg_DN"] is None:
        raise KeyError("the checkpoint has no router weight for this layer")
    return MoE(w["D"], w["H"], w["N"], num_experts_per_tok, 0, save_percent=save_percent,
               bias_update_rate=0.0, Wg_DN=w["Wg_DN"].to(device), Wl1_ND2H=w["Wl1_ND2H"].to(device),
               Wl2_NHD=w["Wl2_NHD"].to(device))


def _stack(t):
    if isinstance(t, torch.Tensor):
        return t
    return torch.stack(list(t))
