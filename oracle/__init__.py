"""Test infrastructure only: CPU restatement of the layer the engine executes.

Nothing under ``kareus_amd/`` imports this package.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` do, and
only as the checker or the timed CPU baseline.
"""
