"""CPU oracle of the GPU-backend hot path.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may import this package; the
product (cinn_amd/) never does.  ``oracle.lib`` binds oracle/libcinn_oracle.so (the C restatement of the
reference's compute definitions, see cinn_oracle.c); ``oracle.ref`` binds oracle/_ref/libcinn_ref_probe.so
(built from the reference's own runtime sources) when it exists.
"""
from .binding import *  # noqa: F401,F403
