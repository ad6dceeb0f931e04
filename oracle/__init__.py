"""CPU oracle for the bidirectional linear-attention operators.

TEST INFRASTRUCTURE ONLY.  Nothing under ``oracle/`` is part of the product:
only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import it, and only as the checker.  The shipped operators
(``flash_bla.ops.*``) never import this package and raise when the HIP library
is missing.

Contents
--------
torch_ref.py    torch restatement of the reference's naive operators
                (flash_bla/ops/linear_attn/naive.py, flash_bla/ops/simple_la/naive.py).
closed_form.py  numpy float64 forward + hand-derived backward for every operator
                family (algebra of flash_bla/ops/linear_attn/fused.py:238-242,325-328,
                decoupled.py:274-283,375-380, varlen.py:216-219,310-314,
                simple_la/fused.py:198,394-397).
piecewise.py    numpy float64 dense evaluation of the piecewise (PISA) forward as
                written in flash_bla/ops/piecewise_attn/kernel.py:105-118,172-176,214-292.
brute.c         plain-C O(L^2) double-precision evaluation of the attention sums,
                no shared algebra with the files above (built into _build/).

Pinning status
--------------
linear_attn / simple_la / decoupled / varlen forward: pinned by brute.c (O(L^2)
pairwise sums), by invariants (constant v, permutation of (k,v) rows, linearity
in v, convex-hull bound, L=1) and by cross-family reductions (decoupled with
q_rope=q reduces to linear_attn, varlen with one sequence reduces to dense).
Backward closed forms: pinned by torch.autograd on torch_ref and by
torch.autograd.gradcheck in float64.
piecewise forward: the reference holds no naive implementation and no test for
it, so its *reference* behaviour is "parity unpinned"; the oracle follows the
kernel text and is pinned mathematically (all blocks selected == softmax
attention; constant keys per chunk make the zeroth-order term exact).
"""
