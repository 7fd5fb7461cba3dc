"""CPU oracle for the TRIM-KV cache hot path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``trimkv_amd/`` may import this package.  It is
used by ``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py`` as the checker / the timed CPU baseline, never as the product path.

Every function restates, with torch CPU ops, what the corresponding function of the
reference (yejun-yun/trimkv, paths relative to its repository root) computes; each one
cites the reference lines it follows.

Pinning status (what independent evidence fixes each function; see tests/test_oracle_*.py):

* dense append / bookkeeping ........ pinned: brute-force concatenation + invariants
* dense eviction (alpha) ............ pinned: numpy full argsort, closed forms
  (equal beta => sliding window, beta ~ 1 never evicted, n == M keeps all)
* dense eviction (knorm_alpha) ...... pinned: numpy float64 norm/log re-derivation + argsort
* flat (ragged) append .............. pinned: per-segment brute force; cu == [0, cumsum(len)]
* ragged eviction (all variants) .... pinned: numpy brute force re-derivation of each variant
  (per-element Python loops on tiny inputs), invariants (popcount == head_lens, order kept)
* eager attention ................... pinned: float64 numpy softmax; one-key and equal-key cases
* ragged decode attention ........... pinned: float64 numpy softmax per segment; the third-party
  flash-attn kernel the reference calls is absent, so agreement with *that* binary is
  "parity unpinned"; the contract is the fp32 eager formula within 2e-2 abs / 1e-2 rel.
* retention gate (rg) ............... pinned: float64 numpy re-derivation (fp32 weights)

``torch.topk`` tie order is a property of the library, not of the reference: parity on the
retained set is defined only when the k-th and (k+1)-th scores differ.
"""
