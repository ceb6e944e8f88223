"""CPU oracle for the MoMoE hot path -- TEST INFRASTRUCTURE ONLY.

This package is a plain restatement, on the CPU, of what the reference computes
for the MoE layer (index build, SwiGLU experts forward/backward, top-k router,
aux-loss-free bias rule).  It exists to check the HIP kernels; it is never part
of the shipped compute path.  Only `tests/`, `__graft_entry__.smoke()` and the
`cpu_baseline` leg of `bench.py` import it.

Pinning status (what makes each function trustworthy without running the
reference, which has no tests, fixtures or golden vectors of its own):

* `index_build`           - pinned: brute-force loops, `numpy.nonzero`,
                            permutation invariants (tests/test_oracle_index.py)
* `experts_forward`       - pinned: dense all-experts evaluation by a different
                            algorithm, N=1/K=1 reduction to a plain SwiGLU MLP
                            built from torch.nn.functional, linearity in s
* `experts_backward_closed_form` - pinned: torch.autograd through
                            `experts_forward` in fp64 and `gradcheck`
* `experts_forward_backward` - pinned: equals `experts_forward` and
                            `experts_backward_closed_form` (tests/test_oracle_experts.py)
* `router_forward`        - pinned: Ks=0/bias=0 reduces to softmax over the
                            top-k logits (library routine); brute-force top-k
* `router_backward_closed_form` - pinned: autograd through a differentiable
                            restatement; finite differences
* `bias_update`           - pinned: closed form on hand-computed cases

The reference's intermediate bf16 rounding points, its autotune-dependent
save/recompute tile boundary and its raced `which` order are NOT restated
(parity unpinned for those three; they are inside the stated tolerance or
explicitly nondeterministic in the reference).
"""
from .moe_oracle import (  # noqa: F401
    index_build,
    index_build_bruteforce,
    experts_forward,
    experts_forward_dense,
    experts_backward_closed_form,
    experts_forward_backward,
    router_forward,
    router_backward_closed_form,
    router_probs_differentiable,
    bias_update,
    OracleMoMoE,
    OracleTopKRouter,
    OracleMoE,
)
