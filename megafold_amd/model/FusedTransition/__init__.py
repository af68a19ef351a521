from .fused_transition import FusedSwiGLU, FusedSwiGLUFunction, FusedTransition  # noqa: F401
