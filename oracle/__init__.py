"""CPU oracle for the quantized MoE expert path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
module; it is the checker used by ``tests/``, ``__graft_entry__.smoke()`` and
the ``cpu_baseline`` leg of ``bench.py``.
"""
