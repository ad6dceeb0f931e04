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
piecewise_tokens.c  plain-C per-token evaluation of the same forward that walks the
                reference kernel's phases (kernel.py:214-292, base-2 running maximum, one
                group) and shares no algebra with piecewise.py; pins its coefficients.
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
it.  piecewise.py is pinned by (i) all blocks selected == softmax attention,
(ii) constant keys per chunk (H = 0) == softmax attention for any selection,
(iii) agreement to 2e-8 with piecewise_tokens.c, a transcription of the kernel
text token by token with one group (where the kernel's un-rescaled g coincides
with the consistent mathematics) on ragged lengths, several block sizes and
explicit scales, with a test that the mistakes G/(T-n_sel), a dropped scale,
a 0.7 factor, a sign and G/NT all fail, and (iv) a zero-mean-chunk case that
isolates the first-order coefficient in closed form with another contraction
order.  What stays open is the Triton kernel's bit-level behaviour with more
than one group (its g is not rescaled, kernel.py:263-276), which is not a
parity target.
"""
