"""Kernel and bias quantizers depend on the variables only (reference src/hgq/layers/core/dense.py:72-79 and the
same lines of the other layers: ``self.kq(self._kernel)``, ``self.bq(self.bias)``), so in a training step all of them
can run in one launch before the first layer, and their gradients in one launch after the last.  A few thousand
elements each, they cost a launch apiece otherwise."""

from __future__ import annotations

import torch

from .. import ops
from .internal.base import bw_layout
from .internal.fixed_point_quantizer import FixedPointQuantizerBase


def _eligible(q, p):
    """The internal quantizer of wrapper ``q`` if its call on parameter ``p`` is exactly one per-element saturating
    quantizer launch, else None."""
    if q is None or p is None or not getattr(q, 'built', False) or not q.plain:
        return None
    fq = q.quantizer
    if not isinstance(fq, FixedPointQuantizerBase) or fq.overflow_mode == 'WRAP' or fq.stochastic:
        return None
    if not (p.is_cuda and p.dtype == torch.float32 and p.is_contiguous()):
        return None
    if fq._i.numel() != p.numel() or bw_layout(fq._i.shape, p.shape) != (p.numel(), 1):
        return None
    return fq


def quantize_together(pairs, training):
    """``[q(x) for q, x in pairs]`` for quantizer wrappers ``q`` and tensors ``x`` (not necessarily variables): one
    launch each way when every pair is a plain per-element saturating quantizer in training mode, else one by one."""
    if training is True and len(pairs) > 1:
        fqs = [_eligible(q, x) for q, x in pairs]
        if all(fq is not None for fq in fqs):
            ys = ops.quantize_multi([x for _, x in pairs], [fq._k.view(-1) for fq in fqs], [fq._i.view(-1) for fq in fqs],
                                    [fq._third().view(-1) for fq in fqs], [fq._mode(True) for fq in fqs])
            return list(ys)
    return [q(x, training=training) for q, x in pairs]


def _plan(root):
    """The layers under ``root`` that declare kernel / bias quantizers; cached on ``root`` until its module tree changes
    (the set of modules and their built flags)."""
    from ..core import tree_cache

    return tree_cache(root).quantized


def prefetch_weight_quantizers(root) -> int:
    """Quantize the kernels and biases of every layer under ``root`` that declares them (``_weight_quantizer_inputs``)
    in one launch and leave each result with its quantizer for the layer's own call to pick up.  Returns the number
    of quantizers served (0: fewer than two were eligible, nothing was done)."""
    pairs = []
    for m in _plan(root):
        if not getattr(m, 'built', False):
            continue
        for q, p in m._weight_quantizer_inputs():
            fq = _eligible(q, p)
            if fq is not None:
                fq._prefetched = None
                pairs.append((fq, p))
    if len(pairs) < 2:
        return 0
    ys = ops.quantize_multi([p for _, p in pairs], [fq._k.view(-1) for fq, _ in pairs], [fq._i.view(-1) for fq, _ in pairs],
                            [fq._third().view(-1) for fq, _ in pairs], [fq._mode(True) for fq, _ in pairs])
    for (fq, p), y in zip(pairs, ys):
        y._hgq_single_use = True  # handed out once, to the layer's own call: the only other reader of its gradient is this launch's backward
        fq._prefetched = (p, y)
    return len(pairs)
