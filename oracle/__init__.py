"""CPU oracle for the attention hot path. TEST INFRASTRUCTURE ONLY.

Nothing in the product package imports this directory. Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
use it, and only as the checker.
"""
