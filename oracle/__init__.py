"""Checker-side Python bindings: TEST INFRASTRUCTURE ONLY.

`port`  - ctypes/numpy wrappers over oracle/libexcalibur_oracle.so, this repository's plain-C
          restatement of the reference's CPU arithmetic (excalibur_oracle.c).
`ref`   - wrappers over oracle/_ref/libexcalibur_ref.so, the reference's own CPU sources compiled by
          oracle/Makefile (present only where that build was made), driven through its public
          pipeline API with hand-written topologies and weight blobs.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this package.
"""
from . import port, ref  # noqa: F401
