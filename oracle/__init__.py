"""CPU oracle for the three fused ops — TEST INFRASTRUCTURE, NOT PRODUCT CODE.

A plain restatement, with stock PyTorch/NumPy on the CPU, of the eager formulas the reference
checks its kernels against.  Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py`` may import this package, and only as the checker / the reported baseline; the
product (``megafold_amd``) never does.

Reference formulas restated here (paths relative to the MegaFold repository):

==========================  =====================================================================
``evoattention``            tests/test_evoattention.py:45-56 (eager attention incl. where the fp32
                            cast happens); benchmarks/evoattention_speed.py:10-16 (bool keep-mask
                            form); megafold/model/attention.py:499-539 (production eager path);
                            gradients: evoattention.py:298, 461-470, 649-661 (closed forms)
``layernorm_linear``        tests/test_layernormlinear.py:17-22; fused_layernorm_linear.py:541
                            (eps, transposed weight); backward: fused_layernorm_linear.py:288-296, 345
``transition``              benchmarks/transition_speed.py:8-39 (SwiGLU half order, module);
                            fused_transition.py:22-24, 44-47 (closed-form derivative)
==========================  =====================================================================

How each function is pinned (the reference ships no golden vectors for these ops; see
``tests/test_oracle_*.py``):

* ``evo_attention_forward``  — equals ``torch.nn.functional.scaled_dot_product_attention`` with the
  additive mask ``bias + res_mask`` (library routine); equals an explicit float64 triple loop on tiny
  shapes; masked keys cannot influence the output; shift invariance; LSE == ``torch.logsumexp``.
* ``evo_attention_backward`` — closed forms equal ``torch.autograd`` of the forward in float64;
  rows of dS sum to zero; masked keys get exactly zero dK/dV/dBias.
* ``layernorm_linear_forward/backward`` — ``F.layer_norm`` + ``F.linear`` (library routines) and their
  autograd in float64; projection identities of the LayerNorm backward.
* ``swiglu_forward/backward``, ``transition_forward`` — ``F.silu`` composition and autograd in
  float64; special values (gate 0, gate -> +inf).
"""
