"""CPU oracle for the MatMul-free LM hot path (BitLinear + HGRN).

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may.  It is the checker, never the thing
measured or shipped.

Two families of functions live here, each citing the reference lines it
follows (paths relative to the reference checkout, package ``mmfreelm``):

* ``*_literal``  -- the reference's PyTorch (non-Triton) formulation, op for op,
  in the tensor dtype the reference would run it in (fake-quantised floats,
  ``F.linear`` on de-quantised weights, torch's own ``sigmoid``/``exp``).
* ``*_spec``     -- the same mathematics with the rounding points of the fused
  device kernels (fp32 math inside a fused op, rounding to the tensor dtype only
  where the reference materialises a tensor, integer-exact contraction, a
  deterministic ``exp`` built from IEEE fp32 add/mul only).  The HIP kernels
  must reproduce ``*_spec`` bit for bit; ``*_spec`` must agree with
  ``*_literal`` to the floating-point tolerance (1e-2 relative in bf16, 1e-3
  with fp32 tensors) and exactly on the int8 / ternary codes wherever both are
  defined on the same fp32 input.

Pinning status (what holds each function to the reference without importing
it; the reference ships no tests, golden vectors or fixtures for this path):

* activation / weight quantisers: closed forms, hand-computed rows with exact
  .5 ties, sign symmetry, scale equivariance, idempotence (tests/test_oracle_quant.py).
* norms, swiglu: fp64 textbook formulas and torch.nn.functional.rms_norm / silu.
* scans: geometric series, cumsum and identity special cases, fp64 brute force,
  split-sequence state carry, chunk == recurrent in exact arithmetic.
* BitLinear: integer-exact identity against an int64 matmul; K=1 and
  identity-like ternary matrices as known answers.
* model wiring: causality / state-carry, batch-row independence, lower-bound
  schedule i/L at zero init.
* The dense contraction inside the reference is ``torch.nn.functional.linear``
  (an unpinned BLAS); no reference test pins its rounding: parity of the
  *float* BitLinear output with the reference's BLAS result is "parity
  unpinned" beyond the stated tolerance; the integer accumulator is exact.
"""
