"""CPU oracle for the HOT linear-layer backward path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package (``hot_amd``) may
import this directory; it is the checker used by ``tests/``, by
``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py``.
"""
