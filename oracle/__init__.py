"""CPU oracle for the mixed-bit MoE routed-expert path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``bitsmoe_amd/`` imports this package; only
``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` do,
and only as the checker / the reported CPU baseline.
"""
