"""CPU oracles for the two hot paths (TEST INFRASTRUCTURE ONLY).

Nothing in the shipped package may import this directory: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` use it,
and only as the checker. The product path is the HIP library and fails loudly
when that library is missing.
"""
