from .pairwise_block import PairwiseBlock  # noqa: F401
