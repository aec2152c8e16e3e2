"""CPU oracle for the MoE hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
directory; only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` do, and there only as the checker.

The reference's implementation of this path is pure Python that delegates all
arithmetic to stock PyTorch ops (pinned torch 2.10), so the restatement is
numpy for the integer routing work and plain CPU torch for the floating-point
expert computation.  Each function cites the reference file:line it follows.

How each function is pinned (the reference ships no golden vectors for this
path, so the pins are what the mathematics fixes; see tests/test_oracle_*.py):

* ``routing.continuous_count``  brute-force Python loop, sum == N, bins == 1
  shortcut, empty bins, torch.bincount.
* ``routing.route``             permutation property, sortedness, strict
  stability inside equal keys, insertion-sort brute force, offsets identities.
* ``moe.swiglu*``               scalar closed form u*g/(1+exp(-g)) evaluated
  with ``math`` on every element; backward against fp64 gradcheck.
* ``moe.routing_weights``       brute-force top-k + softmax per row.
* ``moe.experts_forward``       E=1,k=1 reduces to a dense MLP; all experts
  sharing one weight reduce to the dense MLP for any routing (weights sum to
  1); per-token fp64 brute-force loop; empty experts give zero dW slices.
* backward                      autograd of the fp64 restatement checked with
  finite differences (gradcheck).
"""
