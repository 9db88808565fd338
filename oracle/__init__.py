"""CPU checker for the paged-attention path.  TEST INFRASTRUCTURE, not product.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` import this package, and only to check or to time the CPU side.
``research_amd`` never imports it.
"""
