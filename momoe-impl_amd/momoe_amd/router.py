"""`TopKRouter`: top-k + softmax gate with a selection bias (auxiliary-loss-free load
balancing) and shared experts, mirroring momoe/topk_router.py:83-173.

The gate matmuls are plain library GEMMs (torch); the softmax / top-k / renormalise
pass and its backward are one HIP kernel each.
"""
import torch
import torch.nn as nn

from . import _hip


class TopKRouterFunction(torch.autograd.Function):
    """(x_BSD, Wg_DN, biases_N, N, K, Ks) -> (x_BSD, mask_NM int32 [N,M], s_NM fp32 [N,M]).

    s_NM is the transposed view of an [M,N] matrix, as in the reference
    (momoe/topk_router.py:120); x_BSD is passed through so its gradient picks up
    the gate's contribution (:124, :139).
    """

    @staticmethod
    def forward(ctx, x_BSD, Wg_DN, biases_N, N, K, Ks):
        B, S, D = x_BSD.shape
        M = B * S
        assert Wg_DN.dtype == torch.bfloat16, "Wg_DN must be of type torch.bfloat16"
        dev = Wg_DN.device
        if dev.type != "cuda":
            raise RuntimeError("TopKRouter weights must live on the GPU: there is no CPU compute path")
        with torch.cuda.device(dev):
            x_MD = x_BSD.reshape(M, D).to(device=dev, dtype=torch.bfloat16)
            logits = x_MD @ Wg_DN
            bias = biases_N.to(device=dev, dtype=torch.float32).contiguous()
            mask_NM, s_MN, p_sel_MN, Ng_M, Ks_M = _hip.router_fwd(logits.contiguous(), bias, K, Ks)
        ctx.save_for_backward(x_MD, Wg_DN, mask_NM, p_sel_MN, s_MN, Ng_M, Ks_M)
        ctx.Ks = Ks
        ctx.mark_non_differentiable(mask_NM)
        return x_BSD, mask_NM, s_MN.T

    @staticmethod
    def backward(ctx, G_x_BSD, _, G_s_NM):
        x_MD, Wg_DN, mask_NM, p_sel_MN, s_MN, Ng_M, Ks_M = ctx.saved_tensors
        M, D = x_MD.shape
        dev = Wg_DN.device
        with torch.cuda.device(dev):
            G_x_MD = None
            if G_x_BSD is not None:
                G_x_MD = G_x_BSD.reshape(M, D).to(device=dev, dtype=torch.bfloat16)
            if G_s_NM is None:
                G_Wg = torch.zeros_like(Wg_DN)
                G_x = G_x_MD if G_x_MD is not None else torch.zeros_like(x_MD)
            else:
                G_s = G_s_NM.to(device=dev, dtype=torch.float32)
                G_logit = _hip.router_bwd(G_s, p_sel_MN, s_MN, Ng_M, Ks_M, mask_NM, ctx.Ks)
                if G_x_MD is None:
                    G_x = G_logit @ Wg_DN.T
                else:
                    G_x = torch.addmm(G_x_MD, G_logit, Wg_DN.T)
                G_Wg = x_MD.T @ G_logit
        shape = G_x_BSD.shape if G_x_BSD is not None else (1, M, D)
        return G_x.view(shape), G_Wg, None, None, None, None


class TopKRouter(nn.Module):
    """momoe/topk_router.py:151-173."""

    def __init__(self, embedding_dim, num_experts, num_chosen_experts, num_shared_experts,
                 Wg_DN=None):
        super().__init__()
        self.D = embedding_dim
        self.N = num_experts
        self.K = num_chosen_experts
        self.Ks = num_shared_experts
        if Wg_DN is None:
            Wg_DN = torch.randn((self.D, self.N), device="cuda", dtype=torch.bfloat16) / self.D
        self.Wg_DN = nn.Parameter(Wg_DN.clone().detach().to(torch.bfloat16), requires_grad=True)

    def forward(self, x_BSD, biases_N):
        return TopKRouterFunction.apply(x_BSD, self.Wg_DN, biases_N, self.N, self.K, self.Ks)
