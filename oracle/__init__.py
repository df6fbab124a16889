"""CPU oracle for the block-sparse operator path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``sparta_amd/`` imports this package;
only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may call it, and there only as the checker.  It is a numpy
restatement of the reference's masked-dense semantics; every function cites
the reference file:line it follows.

Pinning status (what fixes each function independently of its own formula):

* ``bcs.reduce_block_mask`` / ``build_bcsr`` / ``build_bcsc`` / ``build_bcsrc``
  - pinned by pure-Python brute force on tiny masks, the all-ones and
  all-zeros closed forms, the bit-field cross-consistency the reference's own
  test decodes (test/unit/test_tesa.py:101-107) and the round trip
  ``get_block_mask() == reduced`` (test_tesa.py:36-38).
* ``bcs.convert`` / ``bcs.inverse`` - pinned by the explicit index formula
  evaluated with Python loops and by the round-trip identity
  (test_tesa.py:41-43).
* ``ops.matmul_reference`` - pinned by triple-loop brute force on tiny inputs,
  all-ones mask == plain GEMM, identity operand == masked copy.
* ``ops.softmax_forward_reference`` / ``softmax_backward_reference`` - pinned by
  all-ones mask == scipy.special.softmax, row sums == 1 on live rows, fully
  masked rows == 0, shift invariance, and a central finite difference for the
  backward.
* ``ops.attention_reference`` - all-ones mask == textbook softmax(QK^T/sqrt(E))V
  evaluated in float64 with loops.
* ``ops.moe_reference`` - single expert == one GEMM; permutation invariance;
  per-token loop brute force.

The reference holds no stored golden vectors for this path (its tests compare
against dense torch on a CUDA device), so there is nothing else to check
against; no function here is "parity unpinned".
"""
