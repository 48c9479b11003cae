"""CPU oracle for the Hadamard hot path -- TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may import
this package, and only as the checker.  The shipped package never imports it.

Two layers:

* ``liboracle.so`` (``hadamard_oracle.c``): plain-C restatement of the reference arithmetic,
  each function citing the reference file:line it follows.
* numpy / torch-CPU helpers below: the reference's own *truth path*, ``x @ (H_n * n**-0.5)``
  with ``H_n = scipy.linalg.hadamard(n)`` (HadaCore/test.py:24-40, bench/bench.py:44-59), and
  the seeded input generators for every benchmark configuration.

The reference's kernels are CUDA (inline PTX, cuBLAS) and cannot be built in this image, so
there is no ``oracle/_ref`` build.
"""
from .oracle import *  # noqa: F401,F403
