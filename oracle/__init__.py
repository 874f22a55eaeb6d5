"""TEST INFRASTRUCTURE: CPU checkers for the decode instruction VM.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package; the shipped ``megakernels_amd`` package
never does.
"""
