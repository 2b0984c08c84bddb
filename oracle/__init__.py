"""CPU oracle for the quantized-matmul hot path (test infrastructure only).

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package; the shipped library never does.
"""
from .oracle import *  # noqa: F401,F403
