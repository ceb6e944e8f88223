"""`MoMoE`: the experts of a SwiGLU mixture-of-experts layer, forward and backward,
on the gfx950 kernels of libmomoe_hip.so.

Mirrors the module and autograd contract of the reference (momoe/momoe.py:847-972):
`MoMoE(embedding_dim, intermediate_dim, num_experts, num_chosen_experts, save_percent,
Wl1_ND2H, Wl2_NHD)`, `forward(x_BSD, mask_NM, s_NM) -> (y_BSD bf16, sizes_N int64)`;
gradients for x (bf16), Wl1/Wl2 (bf16) and s_NM (fp32 [N,M], zero off-mask).

All temporaries are torch allocations made here; the library never allocates.
Nothing in this file synchronises with the device: every launch is sized from
static upper bounds and the routing-dependent tile list lives in device memory.
"""
import torch
import torch.nn as nn

from . import _hip


# The layer requires every token to be routed to exactly K experts (momoe/momoe.py:831, the
# reference's README) and, like the reference, does not verify it: the index build counts the
# offending tokens on the device and reading that counter would stall the host.  With too few
# pairs the missing contributions are simply absent from y and the gradients; with too many (more
# pairs than the M*K sorted rows) the routing is refused on the device: no GEMM runs, y and all
# gradients are zero.  Set CHECK_ROUTING = True to read the counter after
# every forward (one device synchronisation per call) and raise on a violation.
CHECK_ROUTING = False

# Row-tile height of the grouped GEMMs: _hip.AUTO_TILE_ROWS leaves the choice between 256 and 320
# rows to the index build, which makes it on the device from the routing.  A fixed height (a
# multiple of 32 from 32 to _hip.TILE_ROWS) is for experiments and for tests that must cover both code paths.
TILE_ROWS = _hip.AUTO_TILE_ROWS


def _saved_rows(msum, save_percent):
    # momoe/momoe.py:251
    return int(msum * save_percent / 100.0)


class MoEFunction(torch.autograd.Function):
    """(x_BSD, Wl1_ND2H, Wl2_NHD, mask_NM, s_NM, K, save_percent) -> (y_BSD, sizes_N).

    Forward (momoe/momoe.py:856-874): routing index, x.Wl1 with fused SwiGLU,
    h.Wl2 scaled by the gate weight, K-way combine.  With save_percent > 0 the
    pre-activation halves a|b of the first `Msave` sorted rows are kept for the
    backward; everything else is recomputed there.

    Backward (momoe/momoe.py:881-903).  Differences from the reference that do not
    change results beyond rounding: x and G_y are gathered inside the GEMM loads
    instead of being materialised in sorted order; dL/ds is obtained from
    (G_y.Wl2^T).h, which equals G_y.(h.Wl2), so the down projection is never
    recomputed and y_pre is never saved; dL/ds is reduced without atomics.
    """

    @staticmethod
    def forward(ctx, x_BSD, Wl1_ND2H, Wl2_NHD, mask_NM, s_NM, K, save_percent):
        B, S, D = x_BSD.shape
        dev = Wl1_ND2H.device
        assert Wl1_ND2H.device == Wl2_NHD.device, (
            "All weights must be on the same device, but got: Wl1_ND2H.device = {}, "
            "Wl2_NHD.device = {}".format(Wl1_ND2H.device, Wl2_NHD.device))
        if dev.type != "cuda":
            raise RuntimeError("MoMoE weights must live on the GPU: there is no CPU compute path")
        N, Dw, H2 = Wl1_ND2H.shape
        H = H2 // 2
        assert Dw == D and tuple(Wl2_NHD.shape) == (N, H, D)
        M = B * S

        with torch.cuda.device(dev):
            x_MD = x_BSD.reshape(M, D).to(device=dev, dtype=torch.bfloat16).contiguous()
            W1 = Wl1_ND2H.to(torch.bfloat16).contiguous()
            W2 = Wl2_NHD.to(torch.bfloat16).contiguous()
            mask = mask_NM.to(device=dev, dtype=torch.int32)
            s = s_NM.to(device=dev, dtype=torch.float32)

            msum = M * K
            # the Wl1 gradient addresses the eight 32-column blocks of a gz tile with 32-bit byte
            # offsets (momoe_wgrad, k-blocked operand): say so now rather than in the backward
            if ctx.needs_input_grad[1] and 8 * msum * 64 >= 2 ** 32:
                raise RuntimeError(f"MoMoE backward supports fewer than 8388608 (token, expert) pairs per call, "
                                   f"got {msum}: split the batch")
            # nothing is kept for a backward that cannot happen (no input wants a gradient)
            msave = _saved_rows(msum, save_percent) if any(ctx.needs_input_grad[:5]) else 0
            # the backward's recomputing GEMM walks row tiles of its own height: with the height
            # left to the library, the index build writes that table too
            want_rc = any(ctx.needs_input_grad[:5]) and msave < msum and TILE_ROWS == _hip.AUTO_TILE_ROWS
            ib = _hip.index_build(mask, K, tile_rows=TILE_ROWS, recompute_table=want_rc)
            idx, table = ib["idx_Msum"], ib["tile_table"]

            # h in blocks of 32 hidden columns, [H/32][Msum][32]: the layout the down projection reads
            h = torch.empty((H // 32, msum, 32), device=dev, dtype=torch.bfloat16)
            ab_save = torch.empty((msave, 2 * H), device=dev, dtype=torch.bfloat16) if msave > 0 else None
            _hip.lin1_swiglu_fwd(x_MD, W1, idx, table, h, ab_save, 0, msave)
            ys = torch.empty((msum, D), device=dev, dtype=torch.bfloat16)
            _hip.lin2_scale_fwd(h, W2, s, idx, table, ys, M)
            del h
            y_MD = torch.empty((M, D), device=dev, dtype=torch.bfloat16)
            _hip.combine(ys, ib["inv_MK"], y_MD)
            del ys

        ctx.K = K
        ctx.msave = msave
        ctx.has_save = ab_save is not None
        ctx.has_table_rc = want_rc
        saved = [x_MD, s, idx, ib["inv_MK"], ib["cumsums_N"], table, W1, W2]
        if ab_save is not None:
            saved.append(ab_save)
        if want_rc:
            saved.append(ib["recompute_table"])
        ctx.save_for_backward(*saved)
        if CHECK_ROUTING and int(ib["violations"].item()) != 0:
            raise RuntimeError(f"mask_NM: {int(ib['violations'].item())} tokens do not have exactly K = {K} "
                               "experts (or the mask holds more than M*K pairs)")
        sizes_N = ib["sizes_N"]
        ctx.mark_non_differentiable(sizes_N)
        return y_MD.view(B, S, D).to(device=x_BSD.device), sizes_N

    @staticmethod
    def backward(ctx, G_y_BSD, _):
        saved = ctx.saved_tensors
        x_MD, s, idx, inv, cumsums, table, W1, W2 = saved[:8]
        ab_save = saved[8] if ctx.has_save else None
        table_rc = saved[-1] if ctx.has_table_rc else None
        msave = ctx.msave
        B, S, D = G_y_BSD.shape
        M = B * S
        N, H, _ = W2.shape
        msum = idx.numel()
        dev = W1.device
        need_x, need_w1, need_w2, _, need_s = ctx.needs_input_grad[:5]

        with torch.cuda.device(dev):
            Gy = G_y_BSD.reshape(M, D).to(device=dev, dtype=torch.bfloat16).contiguous()

            # dL/dh before the gate weight, in sorted order
            u = torch.empty((msum, H), device=dev, dtype=torch.bfloat16)
            _hip.dgrad_h(Gy, W2, idx, table, u)
            # SwiGLU backward: rows with saved a|b read them; the others recompute a|b = x.Wl1
            # and consume them straight from the GEMM's accumulators
            # G_a|G_b in blocks of 32 columns, [2H/32][Msum][32]: the layout dL/dx contracts over
            gz = torch.empty((2 * H // 32, msum, 32), device=dev, dtype=torch.bfloat16)
            # s*h in groups of 32 padded sorted rows, feature-major inside a group: the layout
            # the Wl2 gradient reads fastest
            hsT = torch.empty((_hip.padded_rows(msum, N) // 32, H, 32), device=dev, dtype=torch.bfloat16)
            nparts = (H + _hip.GS_BLOCK - 1) // _hip.GS_BLOCK
            gs_part = torch.empty((nparts, msum), device=dev, dtype=torch.float32)
            if msave > 0:
                _hip.swiglu_bwd_saved(ab_save, u, s, idx, cumsums, msave, gz, hsT, gs_part)
            if msave < msum:
                # the recomputing GEMM takes shorter row tiles than the others: its own table,
                # from the index build, or made here when the tile height was given
                if table_rc is None:
                    table_rc = _hip.tile_table_build(cumsums, M, ctx.K, _hip.RECOMPUTE_TILE_ROWS)
                _hip.lin1_swiglu_bwd(x_MD, W1, idx, table_rc, u, s, msave, gz, hsT, gs_part)
                del table_rc
            del u

            G_s = None
            if need_s:
                G_s = torch.zeros((N, M), device=dev, dtype=torch.float32)
                _hip.gs_scatter(gs_part, idx, cumsums, G_s)
            del gs_part

            # scratch for the weight gradients of experts with many rows: what the library can
            # use, but no more than u occupied (just freed, so the peak does not move)
            ws_cap = msum * H * 2
            G_W2 = None
            if need_w2:
                G_W2 = torch.empty_like(W2)
                _hip.wgrad(hsT, None, Gy, idx, cumsums, G_W2, M, msum, a_transposed=True,
                           workspace_bytes=min(ws_cap, _hip.wgrad_workspace_bytes(N, H, D, msum)))
            del hsT

            G_W1 = None
            if need_w1:
                G_W1 = torch.empty_like(W1)
                _hip.wgrad(x_MD, idx, gz, None, cumsums, G_W1, M, msum, b_kblocked=True,
                           workspace_bytes=min(ws_cap, _hip.wgrad_workspace_bytes(N, D, 2 * H, msum)))

            G_x_BSD = None
            if need_x:
                gxs = torch.empty((msum, D), device=dev, dtype=torch.bfloat16)
                _hip.dgrad_x(gz, W1, table, gxs, M)
                G_x = torch.empty((M, D), device=dev, dtype=torch.bfloat16)
                _hip.combine(gxs, inv, G_x)
                del gxs
                G_x_BSD = G_x.view(B, S, D).to(G_y_BSD.device)
        return G_x_BSD, G_W1, G_W2, None, G_s, None, None


class MoMoE(nn.Module):
    """Memory-optimised mixture of SwiGLU experts (momoe/momoe.py:914-972).

    Args:
        embedding_dim: D.  intermediate_dim: H.  num_experts: N (shared experts included,
        as the last rows of mask_NM/s_NM).  num_chosen_experts: K per token (shared included).
        save_percent: share of the (token, expert) rows whose pre-activations are kept
        for the backward, 0..100.
        Wl1_ND2H / Wl2_NHD: optional initial weights, [N, D, 2H] and [N, H, D]; the first
        H columns of Wl1 are the linear half, the last H go through SiLU.
    D and H must be multiples of 32 (the k-depth of one GEMM stage).
    """

    def __init__(self, embedding_dim, intermediate_dim, num_experts, num_chosen_experts,
                 save_percent=0, Wl1_ND2H=None, Wl2_NHD=None):
        assert save_percent >= 0 and save_percent <= 100, (
            "save_percent must be between 0 and 100 inclusive, got {}".format(save_percent))
        super().__init__()
        self.D = embedding_dim
        self.H = intermediate_dim
        self.N = num_experts
        self.K = num_chosen_experts
        self.save_percent = save_percent

        if Wl1_ND2H is None:
            Wl1_ND2H = torch.randn((self.N, self.D, 2 * self.H), device="cuda", dtype=torch.bfloat16) / self.D
        if Wl2_NHD is None:
            Wl2_NHD = torch.randn((self.N, self.H, self.D), device="cuda", dtype=torch.bfloat16) / self.D
        self.Wl1_ND2H = nn.Parameter(Wl1_ND2H.clone().detach().to(torch.bfloat16), requires_grad=True)
        self.Wl2_NHD = nn.Parameter(Wl2_NHD.clone().detach().to(torch.bfloat16), requires_grad=True)

    def forward(self, x_BSD, mask_NM, s_NM):
        """x_BSD [B,S,D]; mask_NM int32 0/1 [N,M] with exactly K ones per token; s_NM [N,M]
        gate weights (zero off-mask).  Returns (y_BSD bf16, tokens per expert int64 [N])."""
        # pre-activations are only worth keeping when a backward can follow
        sp = self.save_percent if torch.is_grad_enabled() else 0
        return MoEFunction.apply(x_BSD, self.Wl1_ND2H, self.Wl2_NHD, mask_NM, s_NM, self.K, sp)
