"""CPU oracle for the routed hybrid expert-MLP path -- TEST INFRASTRUCTURE ONLY.

A restatement, in plain PyTorch ops that run on the CPU, of what the reference
computes on this path.  Nothing in ``nestor_amd`` imports it: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may,
and only as the checker.  Every function cites the reference lines it follows
(paths relative to the reference checkout).

Pinning status (what independently fixes each function; see
``tests/test_oracle_pins.py``):

* ``plan.dispatch_plan``      -- brute-force O(rows*E) loop, structural
  invariants, and the input cases of the reference's own map tests
  (tests/test_triton_index_build.py:117-137).  The capacity variant has no
  counterpart on the reference's expert path; it is pinned by its definition
  (brute force) and by reducing to the dropless plan when nothing overflows.
* ``rows.*``                  -- per-row Python loops; finite differences in
  fp64 for the backward formulas; ``F.silu`` / ``torch.cat`` library routines.
  The pool epilogues (``path_mix``, ``path_scale``) and the packed-attention
  epilogue (``gate_combine_slots``) against element loops with hand-placed
  roundings, their backward forms against fp64 autograd of the definition.
* ``bank.segment_mm`` etc.    -- per-expert dense ``matmul`` (the reference's
  own CPU fallback), the sparse per-expert loop, and a per-token loop; the
  biased / pointwise gold against per-token ``F.linear`` on the per-expert
  ``weight`` views.
* ``router.*``                -- ``softmax`` / ``topk`` library routines on
  tie-free inputs, top-1 renorm gate == 1, per-router loop for the batched form;
  the balancing step against a counting loop.

No function of the oracle is "parity unpinned".
"""
