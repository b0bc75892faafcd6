"""MI355X-native ArcticMoE expert layer (gfx950 HIP kernels behind the reference's module surface)."""
from .moe import ArcticMoE, MoEConfig  # noqa: F401

__all__ = ["ArcticMoE", "MoEConfig"]
