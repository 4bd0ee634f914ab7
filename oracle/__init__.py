"""CPU oracle for the RWKV-7 time-mixer path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package imports this directory.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
use it, and only as the checker, never as the thing measured or shipped.

Contents
--------
seq_ref.py      fp64 restatements of the reference's own spec functions
                (the sequential WKV7 recurrence, the attn_ln epilogue, ddlerp,
                expand_loras, the whole TimeMixer forward) plus the naive fp32
                recurrence that serves as the CPU baseline.
chunked_ref.py  fp64 restatement of the chunked algebra (the executable spec
                the HIP kernels were written from), with an optional bf16
                operand-rounding mode that emulates the device arithmetic.
wkv7_oracle.c   the same sequential recurrence in C (fp64) with a hand-derived
                reverse pass, fast enough for the full benchmark shape.
inputs.py       seeded input generators for the tests (bench.py draws the same distributions with builders of its own).

Pinning status (which independent check fixes which function) is listed at the
top of each file.
"""
