"""CPU oracle for the LSH + gated-delta hot path.

TEST INFRASTRUCTURE ONLY. Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package; the shipped ``lampa_amd`` package never does, and it has no CPU
fallback of its own.
"""
