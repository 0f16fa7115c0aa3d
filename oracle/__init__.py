"""CPU oracle for the linear-attention operator path.

TEST INFRASTRUCTURE ONLY.  These modules restate, in plain fp32/fp64 PyTorch on
the CPU, the algorithms the reference pins in its own test files.  They are the
checker for the HIP kernels; nothing in the product package imports them.  Only
``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package.

Parity pin status (what fixes each function independently of its own formula):

* ``gdn.naive_recurrent_gated_delta_rule`` - pinned: agrees with the chunked WY
  composition (a different algorithm), closed forms for beta=0 / K=1, float64
  brute force, chunk-size invariance.
* ``gdn.chunk_local_cumsum`` - pinned against ``torch.cumsum`` on reshaped chunks.
* ``gdn.chunk_scaled_dot_kkt`` - pinned: library matmul + structural zeros.
* ``gdn.solve_tri`` - pinned against ``numpy.linalg.inv`` and the residual test.
* ``gdn.recompute_w_u_fwd`` / ``chunk_fwd_h`` / ``chunk_fwd_o`` - pinned through
  the composition == naive recurrence identity (each stage's omission or sign
  error breaks it) and per-stage library matmuls.
* ``conv1d.causal_conv1d`` - pinned against ``torch.nn.functional.conv1d`` and
  the reference's deterministic arange/128 known-answer inputs.
* ``decode.recurrent_gated_delta_rule`` - pinned against the naive recurrence
  (same maths, different state layout) and the g=None / accepted-token cases.
* ``kda.*`` - pinned: chunked composition == naive per-channel recurrence,
  reduction to GDN when the gate is constant over K, autograd for backward.
"""
