"""CPU oracle for the memorax sequence-model hot path.

TEST INFRASTRUCTURE ONLY.  Nothing under this package is part of the shipped
product: it is imported by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` as the checker / the timed CPU baseline,
never by ``memorax_amd``.

Contents
--------
``oracle.memoroid``   NumPy fp64 restatement of the reference algorithm
                      (reset-aware associative scan over a cell algebra, the
                      diagonal / log-space / additive algebras, linear attention
                      read-out) plus the DeltaNet delta rule, each in several
                      independent formulations that the tests check against each
                      other and against closed forms.
``oracle.grad``       torch-fp64 autograd of the sequential restatements
                      (gradient oracle) and the analytic reverse-scan formulas.
``oracle.c``          plain-C sequential restatement (fwd + analytic bwd),
                      built by ``oracle/Makefile`` into ``oracle/c/libmrx_oracle.so``;
                      used for full-size parity checks and the timed CPU baseline.

Parity pinning status
---------------------
The reference ships no tests, fixtures or golden vectors for this path and its
Python cannot be imported here (JAX/Flax absent), so no function below is
pinned by reference-held vectors: every function is "parity unpinned" with
respect to the reference's own outputs.  Each one is pinned instead by the
mathematics: two or three independent formulations that must agree, closed
forms (cumsum, geometric series, scipy.signal.lfilter, cumprod), brute force on
tiny inputs, associativity / split-invariance / reset-isolation properties and
finite differences for gradients (see ``tests/test_oracle_*.py``).
"""
