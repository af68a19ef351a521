"""MI355X-native (gfx950) replacements for MegaFold's three fused training kernels.

Drop-in operator API, same names and call signatures as the reference:

* ``megafold_amd.model.FusedEvoAttention.evoattention.TritonEvoformer(Q, K, V, res_mask, pair_bias)``
* ``megafold_amd.model.FusedLayernormLinear.fused_layernorm_linear.LayernormLinear(K, N, ...)``
* ``megafold_amd.model.FusedTransition.fused_transition.FusedTransition(dim, expansion_factor, ...)``

Every op runs hand-written HIP kernels through the C ABI in ``include/megafold_amd.h``.
"""
__version__ = "0.1.0"
