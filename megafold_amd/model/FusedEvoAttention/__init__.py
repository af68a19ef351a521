from .evoattention import EvoformerAttention, TritonEvoformer  # noqa: F401
