"""CPU restatement of the MoMoE layer -- TEST INFRASTRUCTURE ONLY (see package docstring).

Everything here is plain numpy / torch on the CPU.  Each function cites the
reference lines whose behaviour it restates (paths relative to the reference
repository root).
"""
from __future__ import annotations

import numpy as np
import torch
import torch.nn as nn
import torch.nn.functional as F


# --------------------------------------------------------------------------
# index build
# --------------------------------------------------------------------------
def index_build(mask_NM) -> dict:
    """Routing index of a 0/1 expert-by-token mask.

    Restates `find_used_experts` + `scatter_cols_kernel`
    (momoe/momoe.py:821-842, 760-815):

    * sizes_N[i]      = number of tokens routed to expert i        (int64, :830)
    * cumsums_N[i]    = exclusive prefix of sizes, cumsums_N[N]=sum (int32, :792-799)
    * idx_Msum[r]     = token id of sorted row r; rows of expert i occupy
                        [cumsums[i], cumsums[i+1]) in ascending token order (:806-810)
    * which_Msum[r]   = slot of that (expert, token) pair among the token's
                        pairs.  The reference assigns slots with a raced
                        atomic counter (:812-813); the value restated here is
                        the one a serial expert-order execution produces:
                        the number of lower-numbered experts that also hold
                        the token.
    * inv_MK[m, k]    = sorted row of token m's k-th pair (inverse of
                        (idx, which); not a reference output, used by the
                        combine step).  -1 where a token has fewer than K pairs.
    """
    mask = np.asarray(mask_NM.cpu() if isinstance(mask_NM, torch.Tensor) else mask_NM)
    assert mask.ndim == 2
    N, M = mask.shape
    set_bits = mask != 0
    sizes = set_bits.sum(axis=1).astype(np.int64)
    cumsums = np.zeros(N + 1, dtype=np.int64)
    np.cumsum(sizes, out=cumsums[1:])
    expert_of_row, idx = np.nonzero(set_bits)  # row-major order: expert asc, token asc
    slots = np.cumsum(set_bits, axis=0) - set_bits  # exclusive count over experts, per token
    which = slots[expert_of_row, idx]
    kmax = int(set_bits.sum(axis=0).max()) if M > 0 and N > 0 else 0
    inv = np.full((M, max(kmax, 1)), -1, dtype=np.int32)
    inv[idx, which] = np.arange(idx.shape[0], dtype=np.int32)
    return {
        "sizes_N": sizes,
        "cumsums_N": cumsums.astype(np.int32),
        "idx_Msum": idx.astype(np.int32),
        "which_Msum": which.astype(np.int32),
        "inv_MK": inv,
        "expert_of_row": expert_of_row.astype(np.int32),
    }


def index_build_bruteforce(mask_NM) -> dict:
    """Same outputs as `index_build`, by explicit loops (small inputs only).

    Follows the serial reading of momoe/momoe.py:790-815: experts in order,
    tokens in order, a per-token counter handing out slots.
    """
    mask = np.asarray(mask_NM.cpu() if isinstance(mask_NM, torch.Tensor) else mask_NM)
    N, M = mask.shape
    sizes = [0] * N
    idx, which, owner = [], [], []
    per_token = [0] * M
    for i in range(N):
        for m in range(M):
            if mask[i, m] != 0:
                idx.append(m)
                which.append(per_token[m])
                owner.append(i)
                per_token[m] += 1
                sizes[i] += 1
    cumsums = [0]
    for c in sizes:
        cumsums.append(cumsums[-1] + c)
    return {
        "sizes_N": np.array(sizes, dtype=np.int64),
        "cumsums_N": np.array(cumsums, dtype=np.int32),
        "idx_Msum": np.array(idx, dtype=np.int32),
        "which_Msum": np.array(which, dtype=np.int32),
        "expert_of_row": np.array(owner, dtype=np.int32),
    }


# --------------------------------------------------------------------------
# experts: forward
# --------------------------------------------------------------------------
def experts_forward(x_MD, Wl1_ND2H, Wl2_NHD, mask_NM, s_NM, dtype=torch.float32,
                    return_intermediates=False):
    """y[m] = sum over experts i holding m of s[i,m] * (a * silu(b)) @ W2_i.

    Per-expert gather loop restating `lin1_kernel` (momoe/momoe.py:108-152:
    `a` is the first H columns of x@W1_i, `b` the last H, activation on `b`),
    `lin2_kernel` (:207-237: down projection then scale by s[i, token]) and
    the sum over the K slots (:290).  Arithmetic is carried out in `dtype`
    (fp32 or fp64); the reference's intermediate bf16 roundings are not
    reproduced.  Differentiable through torch.autograd.
    """
    x = x_MD.to(dtype)
    W1 = Wl1_ND2H.to(dtype)
    W2 = Wl2_NHD.to(dtype)
    s = s_NM.to(dtype)
    N, D, H2 = W1.shape
    H = H2 // 2
    M = x.shape[0]
    y = torch.zeros((M, D), dtype=dtype)
    inter = []
    for i in range(N):
        tok = torch.nonzero(mask_NM[i] != 0, as_tuple=False).flatten()
        if tok.numel() == 0:
            inter.append(None)
            continue
        xi = x.index_select(0, tok)
        z = xi @ W1[i]
        a, b = z[:, :H], z[:, H:]
        h = a * (b * torch.sigmoid(b))
        ypre = h @ W2[i]
        y = y.index_add(0, tok, ypre * s[i].index_select(0, tok)[:, None])
        inter.append((tok, a, b, h, ypre))
    if return_intermediates:
        return y, inter
    return y


def experts_forward_dense(x_MD, Wl1_ND2H, Wl2_NHD, mask_NM, s_NM, dtype=torch.float64):
    """Same function by a different algorithm: every expert applied to every
    token with library ops (einsum + F.silu), then a masked weighted sum.
    Used to pin `experts_forward`."""
    x = x_MD.to(dtype)
    W1 = Wl1_ND2H.to(dtype)
    W2 = Wl2_NHD.to(dtype)
    H = W2.shape[1]
    z = torch.einsum("md,ndh->nmh", x, W1)
    h = z[..., :H] * F.silu(z[..., H:])
    ypre = torch.einsum("nmh,nhd->nmd", h, W2)
    w = (s_NM.to(dtype) * (mask_NM != 0).to(dtype))
    return torch.einsum("nm,nmd->md", w, ypre)


# --------------------------------------------------------------------------
# experts: backward in closed form (the formulas the device kernels implement)
# --------------------------------------------------------------------------
def experts_backward_closed_form(x_MD, Wl1_ND2H, Wl2_NHD, mask_NM, s_NM, G_y_MD,
                                 dtype=torch.float64, reference_rounding=False):
    """Gradients of `experts_forward` written out by hand.

    Restates `swiglu_backward_kernel` (momoe/momoe.py:470-535),
    `weights_update_kernel` (:395-412) and `lin1_backward_kernel` (:662-703):

      Gy' = s * G_y[tok]                      (:340)
      G_h = Gy' @ W2_i^T                      (:475-480)
      G_a = G_h * b * sig(b)                  (:525)
      G_b = G_h * a * sig(b) * (1 + b*(1-sig(b)))   (:526)
      G_W2_i = h^T @ Gy'                      (:593-600)
      G_W1_i = x[tok]^T @ [G_a | G_b]         (:730-737)
      G_x[tok] += [G_a | G_b] @ W1_i^T        (:667-681, :754)
      G_s[i,tok] = sum_d G_y[tok,d] * ypre[d] (:699-703), zero elsewhere (:721)

    `reference_rounding` rounds through bf16 the three intermediates that the
    reference itself stores as bf16 before they enter a weight-gradient GEMM:
    Gy' (:340, the `G_y_MsumD` buffer of :551), the recomputed h (:533-535) and
    G_z (:527-531, `G_z_Msum2H` of :555); the y_pre behind dL/ds is then
    recomputed from that bf16 h, as the reference does for rows without a saved
    y_pre (:689-697; a saved y_pre is bf16 itself).  Everything else stays in `dtype`.
    It exists to measure how far the reference's OWN arithmetic is from the
    unrounded result (tests/test_oracle_experts.py); parity tests compare
    against the unrounded form.
    """
    rnd = (lambda t: t.to(torch.bfloat16).to(dtype)) if reference_rounding else (lambda t: t)
    x = x_MD.to(dtype)
    W1 = Wl1_ND2H.to(dtype)
    W2 = Wl2_NHD.to(dtype)
    s = s_NM.to(dtype)
    Gy = G_y_MD.to(dtype)
    N, D, H2 = W1.shape
    H = H2 // 2
    M = x.shape[0]
    G_x = torch.zeros((M, D), dtype=dtype)
    G_W1 = torch.zeros_like(W1)
    G_W2 = torch.zeros_like(W2)
    G_s = torch.zeros((N, M), dtype=dtype)
    for i in range(N):
        tok = torch.nonzero(mask_NM[i] != 0, as_tuple=False).flatten()
        if tok.numel() == 0:
            continue
        xi = x[tok]
        z = xi @ W1[i]
        a, b = z[:, :H], z[:, H:]
        sig = torch.sigmoid(b)
        h = a * b * sig
        ypre = h @ W2[i]
        gy = Gy[tok]
        gys = rnd(gy * s[i, tok][:, None])
        G_h = gys @ W2[i].T
        G_a = G_h * b * sig
        G_b = G_h * a * sig * (1 + b * (1 - sig))
        G_z = rnd(torch.cat([G_a, G_b], dim=1))
        G_W2[i] = rnd(h).T @ gys
        G_W1[i] = xi.T @ G_z
        G_x.index_add_(0, tok, G_z @ W1[i].T)
        if reference_rounding:
            ypre = rnd(h) @ W2[i]
        G_s[i, tok] = (gy * ypre).sum(dim=1)
    return G_x, G_W1, G_W2, G_s


def experts_forward_backward(x_MD, Wl1_ND2H, Wl2_NHD, mask_NM, s_NM, G_y_MD, dtype=torch.float32):
    """Forward and backward of the experts in one pass over the experts, every product formed
    once: y as in `experts_forward`, the gradients as in `experts_backward_closed_form` (same
    reference lines), with a, b, h and y_pre kept from the forward instead of recomputed -- the
    arithmetic of the reference at save_percent=100, 18*D*H flops per (token, expert) pair.
    No autograd: nothing but the products themselves is executed, which is what a timing of the
    CPU path should measure.  Returns (y, G_x, G_W1, G_W2, G_s)."""
    x = x_MD.to(dtype)
    W1 = Wl1_ND2H.to(dtype)
    W2 = Wl2_NHD.to(dtype)
    s = s_NM.to(dtype)
    Gy = G_y_MD.to(dtype)
    N, D, H2 = W1.shape
    H = H2 // 2
    M = x.shape[0]
    y = torch.zeros((M, D), dtype=dtype)
    G_x = torch.zeros((M, D), dtype=dtype)
    G_W1 = torch.zeros_like(W1)
    G_W2 = torch.zeros_like(W2)
    G_s = torch.zeros((N, M), dtype=dtype)
    for i in range(N):
        tok = torch.nonzero(mask_NM[i] != 0, as_tuple=False).flatten()
        if tok.numel() == 0:
            continue
        xi = x.index_select(0, tok)
        si = s[i].index_select(0, tok)[:, None]
        z = xi @ W1[i]
        a, b = z[:, :H], z[:, H:]
        sig = torch.sigmoid(b)
        h = a * b * sig
        ypre = h @ W2[i]
        y.index_add_(0, tok, ypre * si)
        gy = Gy.index_select(0, tok)
        gys = gy * si
        G_h = gys @ W2[i].T
        G_z = torch.cat([G_h * b * sig, G_h * a * sig * (1 + b * (1 - sig))], dim=1)
        torch.mm(h.T, gys, out=G_W2[i])
        torch.mm(xi.T, G_z, out=G_W1[i])
        G_x.index_add_(0, tok, G_z @ W1[i].T)
        G_s[i, tok] = (gy * ypre).sum(dim=1)
    return y, G_x, G_W1, G_W2, G_s


# --------------------------------------------------------------------------
# router
# --------------------------------------------------------------------------
def router_forward(x_MD, Wg_DN, biases_N, N, K, Ks, logits=None, forced_mask_NM=None):
    """Top-k + softmax router with a selection bias and shared experts.

    Restates `TopKRouterFunction.forward` (momoe/topk_router.py:85-124):
    gate logits are a bf16 x bf16 matmul with bf16 output (:92-95); fp32
    softmax separately over the N-Ks routed columns and the Ks shared
    columns (:97-98); the K-Ks routed experts with the largest
    (probability + bias) are selected (:101); their probabilities are
    renormalised to sum to one (:103-107); shared experts get their group
    softmax divided by its sum (:105,108); mask_NM is int32 with all-ones
    rows for the shared experts (:110-119); s_NM is the transposed view of
    the [M,N] weight matrix (:120).

    `logits` (fp32 [M,N]) may be supplied to bypass the matmul, e.g. to feed
    tie-free fp32 logits.  `forced_mask_NM` replaces the top-k selection by a
    given one (its routed rows): bf16 logits contain exact ties whose order
    torch.topk leaves unspecified, so a test that wants the same routing on
    both sides hands over the selection it checked to be a valid top-k.
    Returns dict with mask_NM, s_NM, p_sel_MN (the masked softmax
    probabilities the backward needs, :106), Ng_M, Ks_M, logits_MN.
    """
    if logits is None:
        logits = (x_MD.to(torch.bfloat16) @ Wg_DN.to(torch.bfloat16))
    M = logits.shape[0]
    Ng = N - Ks
    p_g = torch.softmax(logits[:, :Ng], dim=-1, dtype=torch.float32)
    p_s = torch.softmax(logits[:, Ng:], dim=-1, dtype=torch.float32)
    sel_scores = p_g + biases_N.to(torch.float32)[:Ng][None, :]
    if forced_mask_NM is None:
        _, sel = torch.topk(sel_scores, K - Ks, dim=-1)
        sel_mask = torch.zeros((M, Ng), dtype=torch.bool)
        sel_mask.scatter_(1, sel, True)
    else:
        sel_mask = forced_mask_NM[:Ng].T != 0
    p_sel = p_g * sel_mask
    Ng_M = p_sel.sum(dim=-1)
    Ks_M = p_s.sum(dim=-1)
    s_MN = torch.cat([p_sel / Ng_M[:, None], p_s / Ks_M[:, None]], dim=-1)
    mask_NM = torch.ones((N, M), dtype=torch.int32)
    mask_NM[:Ng] = sel_mask.T.to(torch.int32)
    return {
        "mask_NM": mask_NM,
        "s_NM": s_MN.T,
        "p_sel_MN": torch.cat([p_sel, p_s], dim=-1),
        "Ng_M": Ng_M,
        "Ks_M": Ks_M,
        "logits_MN": logits,
        "sel_scores_MNg": sel_scores,
    }


def router_probs_differentiable(logits_MN, mask_NM, Ks):
    """s_NM as a differentiable function of the logits for a FIXED selection.

    softmax -> constant mask -> renormalise, per group.  Used with autograd to
    pin `router_backward_closed_form`.
    """
    N = mask_NM.shape[0]
    Ng = N - Ks
    sel = (mask_NM[:Ng].T != 0).to(logits_MN.dtype)
    p_g = torch.softmax(logits_MN[:, :Ng], dim=-1)
    p_s = torch.softmax(logits_MN[:, Ng:], dim=-1)
    w_g = p_g * sel
    s_g = w_g / w_g.sum(dim=-1, keepdim=True)
    s_s = p_s / p_s.sum(dim=-1, keepdim=True)
    return torch.cat([s_g, s_s], dim=-1).T


def router_backward_closed_form(G_s_NM, p_sel_MN, s_NM, Ng_M, Ks_M, mask_NM, Ks,
                                round_bf16=False):
    """Gradient of the loss w.r.t. the gate logits, [M,N].

    Restates `normalize_backward_kernel` (momoe/topk_router.py:29-56): per
    token and per group,
        dot   = sum(G_s * s * mask)                 (:39-40)
        out   = (G_s - dot) / group_sum             (:45-46)
        inner = sum(out * p_sel)                    (:49-50)
        G_logit = p_sel * (out - inner)             (:51-52)
    The reference rounds the result through bf16 (:51-56); `round_bf16`
    reproduces that.
    """
    N = mask_NM.shape[0]
    Ng = N - Ks
    dt = G_s_NM.dtype
    g = G_s_NM.T
    s = s_NM.T.to(dt)
    p = p_sel_MN.to(dt)
    msk = (mask_NM.T != 0).to(dt)
    out = torch.zeros_like(g)
    for lo, hi, tot, use_mask in ((0, Ng, Ng_M, True), (Ng, N, Ks_M, False)):
        if hi <= lo:
            continue
        gg, ss, pp = g[:, lo:hi], s[:, lo:hi], p[:, lo:hi]
        mm = msk[:, lo:hi] if use_mask else torch.ones_like(gg)
        dot = (gg * ss * mm).sum(dim=-1, keepdim=True)
        o = (gg - dot) / tot.to(dt)[:, None]
        inner = (o * pp).sum(dim=-1, keepdim=True)
        out[:, lo:hi] = pp * (o - inner)
    if round_bf16:
        out = out.to(torch.bfloat16).to(dt)
    return out


def bias_update(biases_N, sizes_N, M, K, Ks, rate):
    """Aux-loss-free load-balancing step (momoe/sample_moe.py:62-66):
    biases += rate * sign(M*(K-Ks)/(N-Ks) - sizes).  Shared entries are -inf
    and stay -inf (:57)."""
    N = biases_N.shape[0]
    c_avg = M * (K - Ks) / (N - Ks)
    return biases_N + rate * torch.sign(c_avg - sizes_N.to(biases_N.dtype))


# --------------------------------------------------------------------------
# modules with the reference's constructor / forward signatures (CPU, autograd)
# --------------------------------------------------------------------------
class OracleMoMoE(nn.Module):
    """CPU stand-in with the signature of `MoMoE` (momoe/momoe.py:915-972).
    Parameters are kept in `param_dtype`; the forward returns (y_BSD, sizes_N)."""

    def __init__(self, embedding_dim, intermediate_dim, num_experts, num_chosen_experts,
                 save_percent=0, Wl1_ND2H=None, Wl2_NHD=None, dtype=torch.float32):
        super().__init__()
        assert 0 <= save_percent <= 100
        self.D, self.H, self.N, self.K = embedding_dim, intermediate_dim, num_experts, num_chosen_experts
        self.save_percent = save_percent
        self.dtype = dtype
        if Wl1_ND2H is None:
            Wl1_ND2H = torch.randn(self.N, self.D, 2 * self.H) / self.D
        if Wl2_NHD is None:
            Wl2_NHD = torch.randn(self.N, self.H, self.D) / self.D
        self.Wl1_ND2H = nn.Parameter(Wl1_ND2H.clone().detach().to(dtype))
        self.Wl2_NHD = nn.Parameter(Wl2_NHD.clone().detach().to(dtype))

    def forward(self, x_BSD, mask_NM, s_NM):
        B, S, D = x_BSD.shape
        y = experts_forward(x_BSD.reshape(B * S, D), self.Wl1_ND2H, self.Wl2_NHD,
                            mask_NM, s_NM, dtype=self.dtype)
        sizes = (mask_NM != 0).sum(dim=1).to(torch.int64)
        return y.reshape(B, S, D), sizes


class _OracleRouterFn(torch.autograd.Function):
    """Router with the reference's backward (fixed selection, closed form)."""

    @staticmethod
    def forward(ctx, x_BSD, Wg_DN, biases_N, N, K, Ks, forced_mask_NM=None):
        B, S, D = x_BSD.shape
        x_MD = x_BSD.reshape(B * S, D)
        r = router_forward(x_MD, Wg_DN, biases_N, N, K, Ks, forced_mask_NM=forced_mask_NM)
        ctx.save_for_backward(x_MD, Wg_DN, r["mask_NM"], r["p_sel_MN"], r["s_NM"], r["Ng_M"], r["Ks_M"])
        ctx.Ks = Ks
        ctx.mark_non_differentiable(r["mask_NM"])
        return x_BSD, r["mask_NM"], r["s_NM"]

    @staticmethod
    def backward(ctx, G_x_BSD, _, G_s_NM):
        x_MD, Wg_DN, mask_NM, p_sel, s_NM, Ng_M, Ks_M = ctx.saved_tensors
        G_logit = router_backward_closed_form(G_s_NM.to(torch.float32), p_sel, s_NM, Ng_M, Ks_M,
                                              mask_NM, ctx.Ks, round_bf16=True)
        Wg = Wg_DN.to(torch.float32)
        G_x = G_x_BSD.reshape(x_MD.shape).to(torch.float32) + G_logit @ Wg.T
        G_Wg = x_MD.to(torch.float32).T @ G_logit
        return (G_x.reshape(G_x_BSD.shape).to(G_x_BSD.dtype), G_Wg.to(Wg_DN.dtype), None, None, None,
                None, None)


class OracleTopKRouter(nn.Module):
    """CPU stand-in with the signature of `TopKRouter` (momoe/topk_router.py:151-173)."""

    def __init__(self, embedding_dim, num_experts, num_chosen_experts, num_shared_experts, Wg_DN=None):
        super().__init__()
        self.D, self.N, self.K, self.Ks = embedding_dim, num_experts, num_chosen_experts, num_shared_experts
        if Wg_DN is None:
            Wg_DN = torch.randn(self.D, self.N) / self.D
        self.Wg_DN = nn.Parameter(Wg_DN.clone().detach().to(torch.bfloat16))
        self.forced_mask_NM = None  # tests: use this selection instead of torch.topk's

    def forward(self, x_BSD, biases_N):
        return _OracleRouterFn.apply(x_BSD, self.Wg_DN, biases_N, self.N, self.K, self.Ks,
                                     self.forced_mask_NM)


class OracleMoE(nn.Module):
    """CPU stand-in with the signature of `MoE` (momoe/sample_moe.py:16-68):
    router -> experts -> bias update."""

    def __init__(self, embedding_dim, intermediate_dim, num_experts, num_chosen_experts,
                 num_shared_experts, save_percent=0, bias_update_rate=1e-4,
                 Wg_DN=None, Wl1_ND2H=None, Wl2_NHD=None, dtype=torch.float32):
        super().__init__()
        self.D, self.H, self.N = embedding_dim, intermediate_dim, num_experts
        self.K, self.Ks = num_chosen_experts, num_shared_experts
        self.save_percent = save_percent
        self.bias_update_rate = bias_update_rate
        self.router = OracleTopKRouter(self.D, self.N, self.K, self.Ks, Wg_DN=Wg_DN)
        self.momoe = OracleMoMoE(self.D, self.H, self.N, self.K, save_percent,
                                 Wl1_ND2H=Wl1_ND2H, Wl2_NHD=Wl2_NHD, dtype=dtype)
        self.biases_N = nn.Parameter(
            torch.cat([torch.zeros(self.N - self.Ks), torch.full((self.Ks,), float("-inf"))]),
            requires_grad=False)

    def forward(self, x_BSD):
        x_BSD, mask_NM, s_NM = self.router(x_BSD, self.biases_N)
        y_BSD, sizes_N = self.momoe(x_BSD, mask_NM, s_NM)
        B, S, _ = x_BSD.shape
        with torch.no_grad():
            self.biases_N.copy_(bias_update(self.biases_N, sizes_N, B * S, self.K, self.Ks,
                                            self.bias_update_rate))
        return y_BSD
