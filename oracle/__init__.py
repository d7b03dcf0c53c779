"""CPU oracle for the sparse-gradient hot path -- TEST INFRASTRUCTURE ONLY.

Everything under ``oracle/`` is a plain torch-CPU restatement of the
reference's pure-torch path (wenqingqian/SGA: ``sga/kernels_torch.py``,
``sga/plugins/scores.py``, ``sga/plugins/selection/*``, ``sga/support.py``,
``sga/plugins/optimizer/adamw_torch.py``, ``sga/replay.py``,
``sga/replay_fused.py``).  It exists to CHECK the HIP kernels and to serve
as the timed CPU baseline.  It is never the product: only ``tests/``, the
smoke entry and the benchmark's ``cpu_baseline`` leg may import it, and the
``sga_amd`` package never does.

How each function is pinned (what a wrong sign / index / dropped term
would fail) is listed in ``tests/test_oracle_*.py``:

* scores            -- independent float64 closed forms + literal vectors
* k formulas        -- integer closed form, banker's rounding cases
* exact threshold   -- ``torch.kthvalue`` / full sort on adversarial sets
* tie-fill select   -- stable descending sort (first k), reference KATs
* ties-all select   -- ``|s| >= kthvalue``
* balanced select   -- integer closed form on hand-built histograms
* compaction / pack -- ``nonzero`` and brute-force Python loops
* dir table         -- ``torch.searchsorted``
* AdamW commit      -- float64 textbook AdamW, fused-knob == 3-pass identity
* replay commit     -- float64 textbook AdamW/AdamS + dual-lr closed form
* cycle machine     -- T=1 == dense trajectory, from-spec double loop

No function of the oracle is "parity unpinned" except the two build-side
score variants that have no reference counterpart (documented where they
are defined in ``oracle/scores.py``).
"""
