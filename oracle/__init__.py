"""CPU restatement of the YaFSDP per-rank buffer path: TEST INFRASTRUCTURE ONLY.

Nothing in ``yafsdp_amd`` may import this package.  It is the checker used by
``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py``; it is never the thing that is measured as the product or shipped.

Contents
--------
``torch_ops``          the reference's own torch-op sequence (``copy_``, ``split``,
                       ``_foreach_copy_``, ``_foreach_add_``, ``div_``, ``chunk``,
                       ``add_``) run on CPU tensors, each function citing the
                       reference lines it restates.
``layout_bruteforce``  the reference's per-element index method for the ragged
                       split, restated with numpy for tiny inputs.
``bufpath_ref.c``      the same element arithmetic written independently in
                       plain C from the IEEE-754 definitions (integer
                       round-to-nearest-even, true division); built by
                       ``oracle/build.py`` into ``oracle/libbufpath_ref.so``.
``cref``               ctypes loader for the C restatement.

How each function is pinned (the reference ships no tests or golden vectors)
----------------------------------------------------------------------------
* sizing / ragged split: hand-derived known answers and brute force on tiny
  inputs (``tests/test_layout.py``).
* casts: the integer closed form ``(bits + 0x7FFF + ((bits >> 16) & 1)) >> 16``
  and hand-checked tie cases (``tests/test_oracle.py``).
* divide, add, accumulate, rounding order: torch CPU ops versus the C
  restatement versus numpy float64 arithmetic rounded once
  (``tests/test_oracle.py``).
* divide-factor policy: hand-derived table and the upstream twin shipped in the
  installed torch (``tests/test_divide_factors.py``).

The reference package cannot be imported under this interpreter
(``ya_fsdp/_param_group.py:990`` needs Python >= 3.11), so no vector in
``tests/golden`` was produced by running it; the fixtures there come from the
torch-op sequence below and are checked against the independent C restatement.
"""
