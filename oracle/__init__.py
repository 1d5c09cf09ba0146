"""CPU oracle for the per-rank ring-attention step.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; it is used by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` as the checker / reported baseline.
"""
from .ring_oracle import *  # noqa: F401,F403
