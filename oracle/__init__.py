"""TEST INFRASTRUCTURE - CPU oracle of the redistribute path.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this package, and only as the checker.  Nothing under ``etha_amd/`` imports it.

Modules
  dtensor_layout   DTensor's sharding convention restated (which global elements a rank holds)
  reference_path   the reference's Chunk/Bucket byte work restated op for op on torch CPU tensors
  gloo_redistribute  the same with one process per rank and gloo isend/irecv/broadcast as the wire
  c_oracle         ctypes binding of ``reshard_oracle.c`` (casts, gather/scatter, reduce, buckets)
"""
