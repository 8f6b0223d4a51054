"""CPU oracle for the RL training hot path.  TEST INFRASTRUCTURE ONLY.

A plain-PyTorch (CPU, fp32/fp64) restatement of the reference's algorithms for this path.
It exists to check the HIP kernels; nothing under ``areal_amd/`` imports it.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may use it.

Each function cites the reference file:line it follows.  What pins each function (the
reference's own test literals, closed forms, brute force) is listed in the module docstrings
and exercised by ``tests/test_oracle_*.py``.

Parity status:
  * ``oracle.loss.binary_kl`` -- the reference has no test for ``metric="binary_kl"``;
    pinned here by the Bernoulli-KL closed form in float64 and by the fp32 special case
    ``log p = 0`` -> NaN -> token rejected.  Everything else is pinned by re-typed literals of
    the reference's tests.
"""
