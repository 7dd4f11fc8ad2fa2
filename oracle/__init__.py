"""CPU oracle of the AnalogLinear hot path. Test infrastructure only: imported by ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``; never by the product."""
