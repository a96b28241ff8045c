"""Test infrastructure only: CPU restatement of the reference's input layout and channel schedules.

* ``coefficients_to_straight_ref`` follows ``MNIST/dataloader.py:56-61``: a sample is a complex
  vector of ``n_degrees**2`` spherical-harmonic coefficients (degree l occupies entries
  ``l*l .. (l+1)*(l+1)-1``, order m = -l..l, one channel); the network input is the float32
  "straight" array ``(n_degrees**2, 2)`` of (re, im) pairs, degree after degree.
* ``tau_schedule_ref`` follows ``MNIST/model.py:18-28``.

Pinned in tests/test_data_format.py against hand-written small cases (the layout is a pure
re-indexing, the schedules are closed forms).
"""
import math

import numpy as np


def coefficients_to_straight_ref(coefs, n_degrees):
    """One sample (complex vector) or a batch (N, n_degrees**2) -> float32 (..., n_degrees**2, 2)."""
    coefs = np.asarray(coefs)
    single = coefs.ndim == 1
    batch = coefs[None] if single else coefs
    out = []
    for x in batch:
        pairs = np.stack([x.real, x.imag], 1)[None]                 # (1 channel, n, 2)
        rows = [pairs[:, l * l:(l + 1) * (l + 1), :].reshape(-1, 2) for l in range(n_degrees)]
        out.append(np.concatenate(rows).astype(np.float32))
    out = np.stack(out)
    return out[0] if single else out


def tau_schedule_ref(mode, param, lmax):
    """Channels per degree l = 0..lmax for the three schedules of the reference's MNIST model."""
    if mode == 1:
        return [param for _ in range(lmax + 1)]
    if mode == 2:
        return [int(math.ceil(param / (2 * l + 1.0))) for l in range(lmax + 1)]
    if mode == 3:
        return [int(math.ceil(param / math.sqrt(2 * l + 1.0))) for l in range(lmax + 1)]
    raise ValueError("only defined 3 modes: 1,2,3")
