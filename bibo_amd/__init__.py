"""bibo_amd: BiBo's sparse-MoE feed-forward block on hand-written HIP kernels for MI355X (gfx950)."""
from .config import BiBoMoEConfig
from .moe import BiBoFusedExperts, BiBoMoELayer, BiBoMoERouter

__all__ = ["BiBoMoEConfig", "BiBoMoERouter", "BiBoFusedExperts", "BiBoMoELayer"]
