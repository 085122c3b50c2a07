"""CPU/GPU-agnostic plain-torch restatement of the reference's attention operators.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this directory: it is the
checker used by ``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py``.  The product path (``flagattention_amd``) calls hand-written HIP kernels through a
C-ABI library and raises when that library is missing.

Each function follows one file of the reference's PyTorch restatements
(``src/flag_attn/testing/{flash,piecewise,paged}.py``) and cites the lines it follows.

How each function is pinned (the reference ships no golden vectors, every one of its tests is a
randomized three-way comparison), see ``tests/test_oracle_*.py``:

* ``flash_attention``: ``torch.nn.functional.scaled_dot_product_attention`` (non-causal, and
  causal with equal lengths), an explicit fp64 triple loop on tiny inputs (bottom-right causal
  alignment, empty rows), ``torch.logsumexp`` for the log-normalizer, column sums and the
  ``sum_n tot[n] == number of non-empty rows`` invariant for total attention, GQA == MHA on
  repeated heads, closed-form gradients and ``torch.autograd.gradcheck`` in fp64.
* ``piecewise_attention``: reduces to ``flash_attention`` when both (q, k) pairs are equal, when
  the threshold exceeds every distance, when it is below every distance; fp64 loop on tiny inputs;
  closed-form gradients (``src/flag_attn/testing/piecewise.py:36-78``).
* ``paged_attention``: equals dense single-query attention on the gathered keys/values, invariant
  under a permutation of the cache blocks with the block table permuted alike; fp64 loop.

* ``dropout.keep_mask`` (+ the ``dropout_mask`` argument of ``flash_attention``): Philox-4x32 against
  the Random123 known-answer vectors, the uniform map against its defining properties, the drop
  rate, Triton's ``tl.rand`` and the reference's recomputed masks bit for bit; dropout with an all-true
  mask equals no dropout; a hand-built mask against an explicit loop.

All three operators are also held against fixed vectors (``tests/golden/attention_vectors.npz``, written by
``tests/golden/make_vectors.py`` from scalar fp64 loops that state the definitions directly): bottom-right
causal alignment with grouped heads, rows without keys, the piecewise distance rule, the paged block
table (``tests/test_golden.py``; the same vectors check the kernels in the simulator and on the GPU).

No function of this oracle is "parity unpinned".  ``dropout.keep_mask`` in particular reproduces, bit for
bit, Triton's ``tl.rand`` and the masks of the reference's ``recompute_mask_kernel`` (run with Triton's CPU
interpreter; ``tests/golden/dropout_vectors.npz``).
"""
from .flash import flash_attention  # noqa: F401
from .piecewise import piecewise_attention, piecewise_attention_grad  # noqa: F401
from .paged import paged_attention  # noqa: F401
from .compare import max_abs_diff, within_two_x  # noqa: F401
from .dropout import keep_mask  # noqa: F401
