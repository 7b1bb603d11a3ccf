"""CPU oracle for un-normalised causal linear attention, O = tril(Q K^T) V.

TEST INFRASTRUCTURE ONLY.  Nothing in ``flashy_linear_attention_amd`` may import
this package: it exists so that ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` have an independent statement of the
mathematics to check the HIP kernels against.  It is never the thing measured
as the product and never a fallback.

Two restatements live here:

* ``oracle.naive``  -- PyTorch/numpy on the CPU (fp32 or fp64).  Follows the
  naive formula the reference's tests compare against
  (flashlinear/test_attn.py:49-62) and the gradient formulas the reference's
  backward kernel evaluates tile by tile
  (flashlinear/kernels/linear_attn_kernels.py:179-197, 291-299).
* ``oracle/oracle.c`` -- dependency-free C, double accumulation, triple loops
  (built by ``oracle/Makefile`` into ``oracle/_build/liboracle.so`` and loaded
  by ``oracle.c_oracle``).  Used to check the C ABI without torch and as a
  second, independently written opinion on ``oracle.naive``.

Parity status: every function is pinned by ``tests/test_oracle.py`` through
closed forms, invariants, brute force and cross-checks between independently
written forms (masked matmul / prefix-state recurrence / C triple loop /
autograd / finite differences).  The reference stores no golden vectors for
this path (its tests draw inputs at run time on a GPU), so none are checked.
"""
