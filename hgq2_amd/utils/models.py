"""Builders for the synthetic benchmark / parity models."""

from __future__ import annotations

from ..config import LayerConfigScope, QuantizerConfigScope
from ..core import Sequential, set_default_device
from ..layers import QDense


class _Scopes:
    """The scope stack of the reference's README example (README.md:57-67): KBI SAT_SYM
    everywhere, then KIF WRAP on the data lanes, EBOPs on."""

    def __init__(self, beta0):
        self.scopes = [
            QuantizerConfigScope(place='all', default_q_type='kbi', overflow_mode='SAT_SYM'),
            QuantizerConfigScope(place='datalane', default_q_type='kif', overflow_mode='WRAP'),
            LayerConfigScope(enable_ebops=True, beta0=beta0),
        ]

    def __enter__(self):
        for s in self.scopes:
            s.__enter__()

    def __exit__(self, *a):
        for s in reversed(self.scopes):
            s.__exit__(*a)


def qdense_mlp(dims=(16, 64, 32, 32, 5), beta0=1e-5, device=None, batch=None):
    """QDense MLP ``dims[0] -> ... -> dims[-1]`` with ReLU on the hidden layers and a linear output."""
    if device is not None:
        set_default_device(device)
    with _Scopes(beta0):
        layers = [QDense(d, activation='relu' if n < len(dims) - 2 else None) for n, d in enumerate(dims[1:])]
    model = Sequential(layers)
    shape = (batch, dims[0])
    for layer, d in zip(layers, dims[1:]):
        layer._build_device = None
        layer.build(shape)
        layer.built = True
        shape = (batch, d)
    return model
