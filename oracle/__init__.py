"""Test infrastructure: CPU parity checker for the transducer-loss path.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package.  The shipped package
``optimized_transducer_amd`` never does.
"""
