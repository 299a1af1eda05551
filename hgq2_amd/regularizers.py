"""Bit-width regularizers (reference src/hgq/regularizers/__init__.py:8-17)."""

from __future__ import annotations

import torch

__all__ = ['MonoL1', 'Regularizer']


class Regularizer:
    def __call__(self, x):
        return 0.0

    def get_config(self):
        return {}


class MonoL1(Regularizer):
    """``l1 * sum(x)`` (no absolute value: bit-widths are pushed down monotonically)."""

    def __init__(self, l1):
        self.l1 = float(l1)

    def __call__(self, x):
        return self.l1 * torch.sum(x)

    def get_config(self):
        return {'l1': self.l1}
