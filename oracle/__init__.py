"""CPU oracle for sparse entmax attention and entmax rows.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; it is used by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` as the checker / the timed CPU baseline.

Two layers:

* ``oracle.exact``  -- the *exact* alpha-entmax (sort based closed forms for
  alpha = 2 and alpha = 1.5, fp64 bisection for any other alpha) and the dense
  attention built on it, following the semantics of the reference's
  ``examples/attention.py:34-91`` (``slow_entmax_attention``) and of the dense
  references inside ``tests/test_adasplash_v2.py:54-78`` and
  ``tests/test_adasplash.py:24-62``.
* ``oracle.ref_solver`` -- a numpy restatement of the reference's *iterative*
  threshold solvers (``adasplash/triton_entmax_v2.py:43-536``,
  ``adasplash/adasplash_v2.py:69-90,273-289,434-461,563-611`` and
  ``adasplash/adasplash_block_mask.py:15-36,167-175``) acting on dense score
  rows, used to check that those iterates stay inside the stated tolerances of
  the exact answer.

Pinning status (what independent evidence each function is checked against in
``tests/test_oracle.py``):

* ``sparsemax_rows``, ``entmax15_rows``, ``entmax_bisect_rows``,
  ``entmax_rows``: pinned -- variational definition (maximiser of
  ``p.z + H_alpha(p)`` on the simplex, checked against random feasible points
  and scipy's SLSQP), closed forms for 2-element rows, constant rows, one-hot
  rows, the softmax limit alpha -> 1, shift invariance and permutation
  equivariance, and cross-agreement of the three independent algorithms.
* ``dense_entmax_attention``: pinned -- the reference's own known-answer tests
  (q = k = 0, v = 1 -> mean of v, ``tests/test_adasplash.py:173-184``; padded
  rows exactly zero, ``:187-201``), GQA == repeat_interleave
  (``tests/test_adasplash_v2.py:340-342``), varlen == per-batch slicing
  (``:67-78``), and a brute-force per-row loop.
* ``ref_solver.*``: the reference holds no stored vectors for its iterates and
  cannot be executed here (its kernels need CUDA-only Triton externs), so the
  *iterates* are "parity unpinned"; they are only required to land within the
  reference's own test tolerances of the exact answer, which is checked.
"""
