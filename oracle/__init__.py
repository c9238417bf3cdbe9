"""TEST INFRASTRUCTURE -- CPU oracle for the aggregation hot path.

Nothing under ``gnn_benchmark_amd/`` imports this package.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` do, and
only as the checker / the reported CPU baseline.
"""
