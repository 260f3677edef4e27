"""Region-backend side callers of the attention kernel (counterpart of reference backends/)."""
from .transformer_hip import HipTransformerLowering

__all__ = ["HipTransformerLowering"]
