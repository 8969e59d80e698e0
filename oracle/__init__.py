"""CPU oracle for ragged paged attention.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
directory: it is the checker used by ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py``.  The product path is the HIP
library and must fail loudly when that library is missing.
"""
