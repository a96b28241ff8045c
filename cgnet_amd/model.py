"""Classifier on top of the Clebsch-Gordan stack with the reference's module names
(``MNIST/model.py:18-67``): ``SphericalCNN`` -> ``bm1`` (BatchNorm1d) -> ``fcs`` (+ ``dropout_layers``)
-> ``final`` -> log-softmax, so a reference checkpoint's keys load unchanged."""
import functools
import math

import torch
from torch import nn

from . import CGNet


@functools.lru_cache(10)
def define_taus(mode, param, lmax):
    """Channels per degree: 1 constant, 2 ~ param/(2l+1), 3 ~ param/sqrt(2l+1) (rounded up)."""
    if mode == 1:
        return [param for _ in range(lmax + 1)]
    if mode == 2:
        return [int(math.ceil(param / (2 * l + 1.0))) for l in range(lmax + 1)]
    if mode == 3:
        return [int(math.ceil(param / math.sqrt(2 * l + 1.0))) for l in range(lmax + 1)]
    raise ValueError("only defined 3 modes: 1,2,3")


class MNIST_Net(nn.Module):
    def __init__(self, lmax, tau_type=3, tau_man=12, nlayers=5, skipconn=True, norm=True, cuda=True,
                 dropout=0.5, nfc=1, sparse=False, device=None):
        super().__init__()
        assert cuda and norm and skipconn, "Do not support these parameters yet"
        taus = define_taus(tau_type, tau_man, lmax)
        taus = [[1 for _ in range(lmax + 1)]] + [taus for _ in range(nlayers)]
        self.SphericalCNN = CGNet.SphericalCNN(lmax, taus, cuda=cuda, norm=norm, skipconn=skipconn,
                                               sparse_flag=sparse, device=device)
        self.bm1 = nn.BatchNorm1d(self.SphericalCNN.output_length) if norm else None
        self.fcs = nn.ModuleList([])
        self.dropout_layers = None if dropout is None else nn.ModuleList([])
        for layer in range(nfc):
            self.fcs.append(nn.Linear(self.SphericalCNN.output_length if layer == 0 else 256, 256))
            if dropout is not None:
                self.dropout_layers.append(nn.Dropout(p=dropout))
        self.final = nn.Linear(256, 10)
        self.to('cuda' if device is None else device)

    def forward(self, x):
        x = self.SphericalCNN(x)
        if self.bm1 is not None:
            x = self.bm1(x)
        for layer in range(len(self.fcs)):
            x = torch.relu(self.fcs[layer](x))
            if self.dropout_layers is not None:
                x = self.dropout_layers[layer](x)
        return torch.log_softmax(self.final(x), dim=1)
