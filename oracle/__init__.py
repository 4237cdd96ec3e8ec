"""CPU oracle for the FlashBias attention path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this directory:
only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` use it, and there only as the checker.

* ``oracle.eager``   -- eager attention with the bias materialised as
  ``q_bias @ k_bias^T`` (restates ``flash_bias/attention_func.py:16-55`` and the
  grad recipe of ``flash_bias/benchmark.py:65-88``).
* ``oracle.blocked`` -- ctypes binding of ``oracle/blocked.c``, a plain-C fp32
  restatement of the tiled recurrences of ``flash_bias/flash_bias_triton.py``
  (forward ``:128-355``, delta ``:358-400``, backward ``:450-869``).

What pins each function (no reference golden vectors exist for this path, the
reference's only check is a print-only script, ``flash_bias/benchmark.py:22-215``):

====================  ========================================================
eager forward / LSE   brute-force triple loop on tiny shapes; equality with
                      ``torch.nn.functional.scaled_dot_product_attention`` when
                      the factors are zero; the concat identity of
                      ``flash_bias/attention_func.py:188-237``; ``v == 1 -> o == 1``;
                      invariance under a per-row shift of the bias
eager causal          ``o[:, 0] == v[:, 0]``; changing k/v at j > i leaves o[i]
                      bit-identical; rectangular Lq != Lk against brute force
eager gradients       central finite differences in fp64; closed forms
                      ``dV = P^T dO``, ``dS = P*(dP - delta)``, ``dQ = scale dS K``,
                      ``dK = scale dS^T Q``; ``dq_bias = dBias k_bias`` and
                      ``dk_bias = dBias^T q_bias`` (``benchmark.py:76-77``);
                      rows of dS sum to zero
blocked C fwd / bwd   the eager oracle on the fp32 plumbing configuration and
                      on ragged / causal / masked shapes
====================  ========================================================
"""
