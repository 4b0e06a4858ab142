"""CPU oracle for the forward-Laplacian hot path.  TEST INFRASTRUCTURE ONLY.

This package is a plain numpy restatement of the rules that microsoft/folx applies
to the ``(x, jacobian, laplacian)`` triplet.  Nothing in ``folx_amd`` may import it:
only the test-suite, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` use it, and only as the checker or as the reported CPU baseline.

Layout used everywhere in this package (the same as the product's):
  x   : (B, *shape)      value per walker
  J   : (P, B, *shape)   Jacobian rows, Jacobian axis leading (reference ``JAC_DIM = 0``,
                         folx/api.py:16) and the walker axis right behind it
  lap : (B, *shape)      Laplacian per walker

Pinning status (what fixes each function independently of its own formula):
  rules.ACTIVATIONS          closed forms checked against torch fp64 jvp-of-jvp
  rules.dense_rule           brute-force fp64 Hessian trace of small MLPs
  rules.binary rules         brute-force fp64 Hessian trace
  rules.atan2_rule, pow_rule, rem_rule (closed-form gradients and Hessians)
                             brute-force fp64 Hessian trace of torch.atan2 / pow / fmod over all
                             four quadrants and both operand orders
  rules.slogdet_rule         numpy.linalg fp64 + brute-force Hessian trace (n <= 6),
                             diagonal / triangular closed forms, row-swap sign
  rules.inv_rule, solve_rule brute-force fp64 Hessian trace through an adjugate/determinant
                             inverse (cases of test/test_layers.py:443-499), closed forms
  rules.sparse_slogdet_rule, index_algebra.slogdet_*
                             path choices and table shape the reference's tests expect
                             (test/test_layers.py:341-421) + equality with slogdet_rule
  rules.scatter_rule, minmax_rule, index_algebra.scatter_out_mask
                             brute-force fp64 Hessian trace on the cases of
                             test/test_scatter.py; hand-derived masks
  rules.mhsa_rule            brute-force fp64 Hessian trace of softmax(q k^T) v composed
                             with random linear maps, incl. the padded-sequence masks of
                             test/experimental/pallas/test_attention.py:320-326
  index_algebra.find_out_idx the 14 exact-integer cases of test/test_find_out_idx.py
  index_algebra (rest)       brute-force set enumeration on small masks
  parity unpinned            bit-level fp32 rounding of XLA's dots/reductions (the
                             reference pins nothing below rtol 2e-5 either), and the
                             flax ``lecun_normal`` draws of the README MLP configurations (need jax)
"""
