from .fused_layernorm_linear import LayernormLinear, LayernormLinearFunction  # noqa: F401
