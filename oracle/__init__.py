"""TEST INFRASTRUCTURE ONLY -- CPU restatements used as the parity checker.

Nothing in the product (``triturus_amd/``, ``triturus/``) may import this
package.  Allowed users: ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``.

Modules
    oracle64        float64 restatement of the torch recipes that are the
                    reference's own ground truth (baselines/lm2exp.py:11-14,
                    baselines/lt2exp.py:15-25) plus independent closed forms
                    (log-sum-exp over the contracted axes) that pin them.
    torch_baseline  the same recipes in fp32, op for op: the CPU competitor
                    that the benchmark times on the host cores.
    oracle_c        the same path restated in plain C (oracle_c.c: scalar loops,
                    double precision, libm only; built by build_c.py with gcc),
                    reached through ctypes.  Shares no code with oracle64.
    max_ref         first-occurrence arg-max / max with torch's NaN rule,
                    brute force in NumPy (the reference tests use torch.amax /
                    torch.max, tests/max.py:13,22,32).

Pinning status (see tests/test_oracle.py): every function here is checked
against an independent formulation -- the C restatement against the torch one, scipy's logsumexp over the broadcast
R x I x J x K (or R x S x I x J x K) tensor, pure-Python ``math.fsum`` loops on
tiny inputs, and the algebraic special cases (identity a, J = 1, constant b,
column-shift equivariance, rank-1 w).  No function is "parity unpinned".
The reference holds no golden vectors or fixtures for this path (its tests
draw fresh random inputs, tests/lm2exp.py:13-15), so none could be checked.
"""
