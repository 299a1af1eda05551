"""Training-step plumbing for models built from the quantized layers: loss assembly, the SGD
update with the bit-width constraints folded in, and HIP-graph capture of a whole step.

What a Keras trainer does around the layers (reference call stack: tests/base.py:302-321):
sum the user loss, the ``add_loss`` terms (EBOPs * beta) and the variable regularizers; back-
propagate; ``w <- w - lr * g``; apply each variable's constraint.
"""

from __future__ import annotations

import torch

from . import ops
from .regularizers import MonoL1


def model_loss(model, base_loss, fold_regularizers: bool = False):
    """``base_loss + sum(add_loss terms) (+ variable regularizers)``.  With ``fold_regularizers``
    the MonoL1 terms are left out of the autograd graph: their constant gradient ``l1`` is added by
    :class:`SGD` inside the update kernel instead (same update, one launch less per variable)."""
    loss = base_loss
    for m in model.modules():
        for term in getattr(m, '_losses', ()):
            loss = loss + term
    for p in model.parameters():
        r = getattr(p, 'regularizer', None)
        if r is None or not p.requires_grad:  # Keras regularises trainable variables only
            continue
        if fold_regularizers and isinstance(r, MonoL1):
            continue
        loss = loss + r(p)
    return loss


class SGD:
    """Plain SGD (the optimizer of the reference's training test, tests/base.py:313) with the
    per-variable constraint applied after the update, as Keras optimizers do."""

    def __init__(self, params, lr: float = 0.01, fold_regularizers: bool = False):
        self.params = [p for p in params if p.requires_grad]
        self.lr = float(lr)
        self.fold_regularizers = fold_regularizers

    def zero_grad(self, set_to_none: bool = True):
        for p in self.params:
            if set_to_none:
                p.grad = None
            elif p.grad is not None:
                p.grad.zero_()

    @torch.no_grad()
    def step(self):
        ws, gs, l1s, los, his, post = [], [], [], [], [], []
        for p in self.params:
            if p.grad is None:
                continue
            c = getattr(p, 'constraint', None)
            r = getattr(p, 'regularizer', None)
            bounds = c.bounds() if c is not None else (float('-inf'), float('inf'))
            if bounds is None:  # a constraint that is not a clip: applied after the update
                bounds = (float('-inf'), float('inf'))
                post.append((p, c))
            ws.append(p.data)
            gs.append(p.grad)
            l1s.append(r.l1 if (self.fold_regularizers and isinstance(r, MonoL1)) else 0.0)
            los.append(bounds[0])
            his.append(bounds[1])
        if ws:
            ops.sgd_update_multi_(ws, gs, l1s, los, his, self.lr)
        for p, c in post:
            p.copy_(c(p))


class GraphedTrainStep:
    """One training step (forward, loss, backward, optimizer update) captured in a HIP graph.

    The step is launch-bound at the layer sizes this package targets (tens of small kernels), so
    the whole sequence is recorded once on a side stream and replayed; inputs are copied into
    static buffers before each replay.  ``loss_fn(outputs, labels)`` must be built from capturable
    operations (``hgq2_amd.ops.sparse_ce`` is)."""

    def __init__(self, model, loss_fn, optimizer: SGD, example_x, example_y, warmup: int = 3):
        self.model, self.loss_fn, self.opt = model, loss_fn, optimizer
        self.x = example_x.clone()
        self.y = example_y.clone()
        self.loss = None
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(warmup):
                self._step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.opt.zero_grad(set_to_none=True)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.loss = self._step()

    def _step(self):
        self.opt.zero_grad(set_to_none=True)
        out = self.model(self.x, training=True)
        loss = model_loss(self.model, self.loss_fn(out, self.y), self.opt.fold_regularizers)
        loss.backward()
        self.opt.step()
        return loss.detach()

    def __call__(self, x=None, y=None):
        if x is not None:
            self.x.copy_(x)
        if y is not None:
            self.y.copy_(y)
        self.graph.replay()
        return self.loss
