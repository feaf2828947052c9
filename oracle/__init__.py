"""CPU oracle for the g4b attention hot path.

TEST INFRASTRUCTURE ONLY.  Nothing under this package is part of the product: it
is imported by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` as the checker / the timed CPU baseline,
never by ``g4b_amd``.  The product path calls hand-written HIP kernels through a
C ABI and raises when that library is missing.

Contents
--------
``index_spec``     integer contracts: ring slot mapping, window bounds, stage and
                   split ranges, KV-append rows, scheduler integers, split
                   heuristic (reference ``g4b/kernels/fa2.py``,
                   ``g4b/kernels/add_kv_to_cache.py``, ``g4b/scheduler.py``,
                   ``g4b/models/gemma4e.py``).
``attention_ref``  floating-point restatements: dense masked softmax attention in
                   fp64 (the parity oracle), the torch-CPU fp32 restatement of
                   ``scripts/reference_impl.py:421-443`` (the timed CPU baseline),
                   a tile-by-tile restatement of the Triton program
                   (``g4b/kernels/fa2.py:37-136,322-480``) and of the split merge
                   (``:546-631``), KV append and decode-state advance.

Pinning status (each item is checked in ``tests/test_oracle_*.py``)
-------------------------------------------------------------------
The reference holds no golden vectors for this path (its compare scripts draw
unseeded random inputs and print differences).  Every oracle function is pinned
by checks that do not retype its formula:

* ``attention_ref``: against ``torch.nn.functional.scaled_dot_product_attention``
  on CPU with an explicit boolean mask built from *absolute positions* of a
  simulated token stream appended to a ring (not from the window formulas);
  exact special cases (all-zero K gives the mean of the visible V rows, which
  reads back the visible set exactly; one dominant key returns that V row).
* ring / window / stage / split integers: brute force over all small
  ``(tds, W, KV_CTX, Tq, BM, S)`` against the position model, and against the
  reference test's own one-liner ``roll(x, -ring_start)[:, :window]``
  (``tests/compare_scripts/test_fa2.py:128-132``).
* ``flash_tiles_ref`` (the Triton decomposition with additive -1e6 masks and
  exp2) must equal ``attention_ref`` wherever every query row sees a key.
* ``reduce_split_kv_ref``: S-way split then merge equals the unsplit result.
* ``kv_append_ref``: the reference test's one-liner
  ``cache[b,:,(arange(t)+off[b])%T,:] = x[b]`` at its shapes
  ``B,G,t,T,D = 2,4,7,17,256``, offsets ``[15,3]``
  (``tests/compare_scripts/test_add_kv.py:19-59``).
* ``retrieve_ref_torch``: against ``attention_ref`` (two independent codings of
  the same 23 reference lines, one list-sliced like the reference, one masked).

No function is "parity unpinned".
"""
