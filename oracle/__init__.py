"""CPU oracle for the LBI bounded-interface backward hot path.

TEST INFRASTRUCTURE ONLY. Nothing in the shipped package imports this
directory; the only callers are ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``, and there only as the checker or the
timed CPU baseline, never as the product path.

Every function restates, in plain torch / numpy on the CPU, one piece of the
reference algorithm and cites the reference file:line it follows.

Parity status of each oracle function (what pins it, see tests/test_oracle_*.py):

* ``scan.suffix_scan_levels``          pinned: 2x2 known-answer vector of the
  reference tests, fp64 brute-force loops, permutation / diagonal / d=1 closed
  forms, recurrence invariant ``out[r] == mats[r] @ out[r+1]``.
* ``scan.suffix_scan_sequential``      pinned: same vectors and closed forms.
* ``scan.suffix_cotangents_sequential`` pinned: equals suffix matrices applied
  to g; d=1 cumulative product closed form.
* ``attention.attention_pullback_dense`` pinned: torch SDPA + autograd (library
  routine the reference tests use as their own oracle), central finite
  differences in fp64, hand-computed T=1 / T=2 closed forms, invariants.
* ``attention.attention_pullback_sdpa_loop`` pinned: agreement with the dense
  formula and the finite differences.
"""
