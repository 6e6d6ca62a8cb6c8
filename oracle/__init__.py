"""CPU oracle for the draft-model training hot path.

TEST INFRASTRUCTURE ONLY.  This package restates, in plain fp32 PyTorch / numpy
on the CPU, the algorithm of the reference path (vllm-project/speculators,
``src/speculators/models/{eagle3,dflash}``, ``src/speculators/losses``,
``src/speculators/models/metrics.py``).  It is the checker the HIP kernels are
compared with; nothing in ``speculators_amd`` imports it, and only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may.

Every function cites the reference file:line it follows.  How each function is
pinned (reference golden vectors, closed forms, brute force) is listed in the
docstring of the module that holds it; functions without such a pin say
"parity unpinned".

Parity unpinned: none.  (``losses.dpace_loss_decay`` has no test in the reference; it is
pinned by what its formula fixes: a per-element float64 double loop over random masks.)
"""
