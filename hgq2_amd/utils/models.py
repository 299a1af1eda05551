"""Builders for the synthetic benchmark / parity models."""

from __future__ import annotations

from ..config import LayerConfigScope, QuantizerConfigScope
from ..core import Sequential, set_default_device
from .. import host, ops
from ..core import Layer
from ..layers import QConv2D, QDense, QEinsumDenseBatchnorm, QMultiHeadAttention


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


class Lambda(Layer):
    """A parameter-free step between quantized layers (pooling, flatten, mean)."""

    def __init__(self, fn, host_fn=None, **kwargs):
        super().__init__(**kwargs)
        self.fn = fn
        self.host_fn = host_fn or fn  # the same step on CPU tensors, for checking against the oracle

    def call(self, x, training=None):
        return self.fn(x)


# layers without variables between the quantized ones; each has ``host_fn``, the same step on CPU tensors
PARAMETER_FREE = (Lambda, host.MaxPooling2D, host.AveragePooling2D, host.Flatten, host.GlobalAveragePooling1D)


def particle_mlp(n_particles=64, n_features=16, hidden=(64, 32), n_out=5, beta0=1e-5, device=None):
    """Per-particle network: QEinsumDenseBatchnorm('bpf,fh->bph') x len(hidden) with ReLU, mean over the
    particles, QDense(n_out)."""
    if device is not None:
        set_default_device(device)
    with _Scopes(beta0):
        layers = [QEinsumDenseBatchnorm('bpf,fh->bph', (n_particles, h), bias_axes='h', activation='relu') for h in hidden]
        layers.append(host.GlobalAveragePooling1D(name='mean_over_particles'))
        layers.append(QDense(n_out))
    return Sequential(layers)


def conv_stack(filters=32, n_out=10, beta0=1e-5, device=None):
    """QConv2D 3x3 ReLU -> MaxPool 2x2 -> QConv2D 3x3 ReLU -> Flatten -> QDense(n_out), channels-last."""
    if device is not None:
        set_default_device(device)
    with _Scopes(beta0):
        layers = [QConv2D(filters, (3, 3), activation='relu'), host.MaxPooling2D((2, 2), name='max_pool'),
                  QConv2D(filters, (3, 3), activation='relu'), host.Flatten(name='flatten'), QDense(n_out)]
    return Sequential(layers)


def mha_block(num_heads=4, key_dim=16, beta0=1e-5, device=None):
    """Self-attention block: QMultiHeadAttention with the table softmax (8-bit tables by default)."""
    if device is not None:
        set_default_device(device)
    with _Scopes(beta0):
        layer = QMultiHeadAttention(num_heads=num_heads, key_dim=key_dim)
    return layer
