"""CPU oracle for the pre-tjax kernel path.  TEST INFRASTRUCTURE ONLY.

Nothing under this directory is part of the shipped product: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it, and there only as the checker.  The product (``pre-tjax_amd``)
never imports it and has no CPU fallback.

Each function restates the algorithm of the reference and cites the
reference file:line it follows.  How each function is pinned (closed forms,
library routines, known-answer vectors) is listed in ``tests/test_oracle_*.py``.
"""
