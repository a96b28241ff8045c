"""Input side of the Clebsch-Gordan stack: spherical-harmonic coefficient files -> "straight" batches.

The reference stores one complex coefficient vector per image in ``L_<n>.npy`` (shape
``(N, n*n)``, degree l in entries ``l*l .. (l+1)*(l+1)-1``, see ``MNIST/MNIST_data_process.py:130-151``)
and turns a sample into the float32 array ``(n*n, 2)`` of (re, im) pairs in ``MNIST/dataloader.py:56-61``.
With one channel per degree that array *is* the straight layout the layers take, so the conversion
is a re-interpretation of the complex numbers, done here for whole batches without a python loop.
"""
import numpy as np
import torch
from torch.utils.data import Dataset


def coefficients_to_straight(coefs, n_degrees=None):
    """Complex array (..., n) -> float32 tensor (..., n_degrees**2, 2); ``n_degrees`` truncates to the
    first ``n_degrees**2`` coefficients (a file computed for more degrees can serve fewer)."""
    coefs = np.asarray(coefs)
    if not np.iscomplexobj(coefs):
        raise TypeError("expected complex spherical-harmonic coefficients, got dtype %s" % coefs.dtype)
    if n_degrees is not None:
        if coefs.shape[-1] < n_degrees * n_degrees:
            raise ValueError("%d coefficients cannot hold %d degrees" % (coefs.shape[-1], n_degrees))
        coefs = coefs[..., :n_degrees * n_degrees]
    c64 = np.ascontiguousarray(coefs, dtype=np.complex64)
    return torch.from_numpy(c64.view(np.float32).reshape(c64.shape + (2,)))


class CoefficientFile(Dataset):
    """Samples of a ``L_<n>.npy`` coefficient file (memory-mapped) with optional labels.

    ``__getitem__`` returns ``(x, y, idx)`` like the reference's dataset: ``x`` float32 ``(n_degrees**2, 2)``,
    ``y`` the label (or -1 without a label file)."""

    def __init__(self, coef_path, n_degrees, label_path=None, indices=None):
        self.coefs = np.load(coef_path, mmap_mode='r')
        if self.coefs.ndim != 2 or self.coefs.shape[1] < n_degrees * n_degrees:
            raise ValueError("%s holds shape %s, need (N, >= %d)" % (coef_path, self.coefs.shape, n_degrees ** 2))
        self.labels = None if label_path is None else np.load(label_path)
        if self.labels is not None and len(self.labels) != len(self.coefs):
            raise ValueError("labels and coefficients differ in length")
        self.indices = np.arange(len(self.coefs)) if indices is None else np.asarray(indices)
        self.n_degrees = n_degrees

    def __len__(self):
        return len(self.indices)

    def __getitem__(self, idx):
        if torch.is_tensor(idx):
            idx = idx.tolist()
        if idx >= len(self.indices):
            raise IndexError("%d is out of range (%d elements)" % (idx, len(self.indices)))
        k = int(self.indices[idx])
        x = coefficients_to_straight(np.asarray(self.coefs[k]), self.n_degrees)
        y = -1 if self.labels is None else int(self.labels[k])
        return x, y, idx

    def batch(self, idxs):
        """A whole batch (B, n_degrees**2, 2) in one conversion."""
        ks = self.indices[np.asarray(idxs)]
        order = np.argsort(ks)                                   # ascending reads from the memory map
        rows = np.asarray(self.coefs[ks[order]])
        inv = np.empty_like(order)
        inv[order] = np.arange(len(order))
        return coefficients_to_straight(rows[inv], self.n_degrees)
