"""CPU oracle for the fused-attention hot path.  TEST INFRASTRUCTURE ONLY.

Nothing under ``loopfuse_amd/`` imports this package.  It may be imported by
``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py`` -- and there only as the checker / the timed CPU baseline.
"""
