"""CPU oracle for the quantized-inference hot path (test infrastructure only).

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package; the shipped GPU path never does.
"""
from .q8_oracle import *  # noqa: F401,F403
from . import observer_oracle  # noqa: F401,E402
