"""Writes the frozen vectors in this directory.

The reference keeps no golden vectors for this path (its tests draw fresh
random inputs on the GPU, tests/lm2exp.py:13-15, tests/lt2exp.py:19-22), so
these fixtures come from this repository's float64 oracle, after that oracle
has been pinned against the independent closed forms in tests/test_oracle.py.
They freeze small, awkward cases (ragged shapes, -inf entries, an all -inf
column, a zero row of weights, arg-max ties) so that a later change to either
the oracle or the kernels is noticed.

Run from the repository root:  python tests/golden/make_golden.py
"""

import sys
from pathlib import Path

import numpy as np
import torch

HERE = Path(__file__).resolve().parent
sys.path.insert(0, str(HERE.parents[1]))

from oracle import oracle64  # noqa: E402
from oracle.max_ref import matmax_ref, vmax_ref  # noqa: E402


def lm2exp_case(seed, R, I, J, K):
    g = torch.Generator().manual_seed(seed)
    a = torch.rand(R, I, J, generator=g)
    b = -5.0 + 4.0 * torch.randn(R, J, K, generator=g)
    b[torch.rand(b.shape, generator=g) < 0.1] = float("-inf")
    b[0, :, K // 2] = float("-inf")  # all -inf column -> -inf output column
    a[R - 1, I // 2, :] = 0.0  # zero row of weights -> -inf output row
    return a, b


def lt2exp_case(seed, R, S, I, J, K):
    g = torch.Generator().manual_seed(seed)
    w = torch.rand(R, S, I, J, generator=g)
    a = -3.0 + 2.0 * torch.randn(R, I, K, generator=g)
    b = -3.0 + 2.0 * torch.randn(R, J, K, generator=g)
    a[torch.rand(a.shape, generator=g) < 0.1] = float("-inf")
    b[torch.rand(b.shape, generator=g) < 0.1] = float("-inf")
    b[0, :, 1] = float("-inf")
    w[R - 1, S // 2] = 0.0
    return w, a, b


def main():
    out = {}
    for name, (seed, shape) in {
        "lm2exp_small": (101, (2, 5, 7, 9)),
        "lm2exp_ragged": (102, (3, 37, 41, 70)),
    }.items():
        a, b = lm2exp_case(seed, *shape)
        out[name] = dict(a=a.numpy(), b=b.numpy(), c=oracle64.lm2exp64(a, b).numpy())
    for name, (seed, shape) in {
        "lt2exp_small": (201, (2, 3, 4, 5, 6)),
        "lt2exp_ragged": (202, (2, 35, 9, 13, 45)),
    }.items():
        w, a, b = lt2exp_case(seed, *shape)
        out[name] = dict(w=w.numpy(), a=a.numpy(), b=b.numpy(), c=oracle64.lt2exp64(w, a, b).numpy())
    g = torch.Generator().manual_seed(301)
    x = torch.randint(-4, 5, (1000,), generator=g).float()  # many ties
    v, i = vmax_ref(x.numpy())
    out["vmax_ties"] = dict(x=x.numpy(), value=np.float32(v), index=np.int64(i))
    xm = torch.randint(-9, 10, (23, 31), generator=g).float()
    out["matmax_small"] = dict(x=xm.numpy(), axis0=matmax_ref(xm.numpy(), 0), axis1=matmax_ref(xm.numpy(), 1))
    for name, arrays in out.items():
        np.savez_compressed(HERE / f"{name}.npz", **arrays)
        print(name, {k: getattr(v, "shape", ()) for k, v in arrays.items()})


if __name__ == "__main__":
    main()
