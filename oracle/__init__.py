"""CPU oracle for the quantized linear-layer path: test infrastructure only.

Only tests/, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package; the product library never does.
"""
