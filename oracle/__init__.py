"""CPU restatement of the reference's configuration-search path (numpy / plain C).

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package ``mist_amd`` imports, links or runs
anything from this directory; only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` do, and only as the checker.

Each module restates one part of the reference (file:line cited per function):

* ``comm``          alpha-beta GPU<->GPU and CPU<->GPU models   mist/tools/optimize.py:201-303,459-470
* ``interference``  four-resource overlap model                  mist/tools/optimize.py:552-571,951-964,1012-1122
* ``pareto``        alpha-weighted argmin sampling               mist/utils/pareto.py:8-156
* ``search_space``  strategy-row enumeration, mesh / G lists     mist/analyzer/batched_module_analyzer.py:417-536, mist/tuning/optimization.py:30-55
* ``stage``         per-stage latency + memory model + reduction mist/analyzer/batched_module_analyzer.py:581-3144
* ``stage_c``       ``stage``'s (ckpt, pre-saved micro-batch) loops and argmin scan in plain C
                    (``stage_loop.c``, OpenMP; same operations in the same order, held bit-equal
                    to the numpy loops by tests/test_oracle_stage_c.py)   :2218-3106, mist/utils/pareto.py:124-144
* ``intra``         (G, mesh) driver and table packing           mist/analyzer/intra_tuning.py:84-282
* ``inter_dp``      inter-stage DP with t_max enumeration        mist/analyzer/inter_tuning.py:63-355
* ``inter_uniform`` uniform / uniform-device inter-stage search  mist/analyzer/inter_tuning_uniform.py:95-397, inter_tuning_uniform_device.py:69-441

Parity status.  The reference holds no tests, golden vectors or fixtures for any function on
this path, it cannot be imported here (numba, hydra, omegaconf, pulp, more_itertools are
absent) and its traced inputs need a CUDA GPU, so every function is pinned only by what the
mathematics fixes (hand-computed cells typed as literals, closed forms, invariants, brute force
on tiny inputs, numpy library routines); see tests/test_known_answer_cells.py and
tests/test_oracle_*.py.  What none of those can pin is marked "parity unpinned" at the function:
(1) numba ``fastmath`` contraction / reassociation of ``alpha/(1-alpha)*x + y`` for sample sizes
above one (``stage_loop.c`` has a build with the fused form; on every group of the three
smaller benchmark plans with 30 samples it picks the same rows), (2) numpy-1.24 legacy scalar promotion
in the two scalar expressions of the inter-stage scan, which are restated with explicit float64
casts.
"""
