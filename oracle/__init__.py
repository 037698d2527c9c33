"""CPU oracle for the decaying-fast-weight (LFW) and delta-rule (DFW) recurrences.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package (``t2fw_amd``/``t2fw``)
imports this directory; only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` do, and only as the checker.
"""
