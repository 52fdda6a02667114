"""CPU restatement of the reference llama decoder-layer training step.

TEST INFRASTRUCTURE ONLY.  Nothing under ``oracle/`` is part of the shipped
path: only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg
of ``bench.py`` may import it, and only as the checker.
"""
