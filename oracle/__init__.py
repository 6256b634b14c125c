"""CPU oracle: TEST INFRASTRUCTURE ONLY.

A restatement, in numpy, of the reference's own CPU evaluation of the programs on the hot
path.  Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may
import this package, and only as the checker: nothing under ``cleave_amd/`` imports it, and
no kernel launch path can reach it.

* ``program_oracle``: ``Program.reference`` + ``grouped_matmul``
  (reference ``python/cleave/frontend/program.py:296-363``).
* ``paged_oracle``: ``gqa_paged_decode_reference`` with ``_paged_tokens`` / ``_attend`` /
  ``_finish`` (reference ``python/cleave/dynamic/reference.py:62-200``), plus the slab layer's
  ``valid_len`` arithmetic (``python/cleave/dynamic/paging/builders/slab.py:138-142``) and the
  split range arithmetic (``python/cleave/dynamic/paging/stages.py:331-347``).

Parity status.  Every function is pinned by tests under ``tests/test_oracle.py`` against
closed forms the reference's own tests use (``tests/frontend/test_program.py:26-52``,
``tests/frontend/test_exact_softmax.py:34-43``: ``x.float() @ w.float()``, ``xf * rsqrt(mean
xf^2) @ wf``, ``softmax(q k^T / sqrt d) v`` with ``repeat_interleave`` groups), against float64
brute force on tiny inputs, against invariants (softmax shift invariance, page permutation
invariance, every KV tile owned by exactly one split) and against the golden vectors in
``tests/golden/``.  The reference's Python was not imported or run to produce any of them.
The device arithmetic of the reference (TileLang's ``T.gemm``/``T.exp2``) has no CPU
counterpart in the reference tree: parity at that boundary is unpinned, and is instead pinned
one level up, at these torch-level evaluators.
"""
