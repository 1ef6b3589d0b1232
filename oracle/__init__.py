"""CPU restatement of the reference's ONNX expansions: the parity checker.

TEST INFRASTRUCTURE ONLY. Imported by ``tests/``, ``__graft_entry__.smoke()`` and
the ``cpu_baseline`` leg of ``bench.py``; the product package never imports it.
``pure_ops`` is the numpy restatement, ``c_oracle`` loads the C restatement
(``pure_ops.c``, built by ``oracle/Makefile``) that is also timed as the CPU
baseline.
"""
from . import pure_ops  # noqa: F401
