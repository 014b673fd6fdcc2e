"""TEST INFRASTRUCTURE: CPU oracle of the Cascading-KV-Cache hot path.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may import
this package; the product package never does.
"""
