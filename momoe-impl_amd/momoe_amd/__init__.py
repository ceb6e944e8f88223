"""MI355X-native MoMoE: SwiGLU mixture-of-experts layer on hand-written gfx950 kernels.

Same public names as the reference package (momoe/__init__.py:1-5).
"""
from .experts import MoMoE, MoEFunction
from .router import TopKRouter, TopKRouterFunction
from .moe import MoE

__all__ = ["MoMoE", "MoE", "TopKRouter", "MoEFunction", "TopKRouterFunction"]
