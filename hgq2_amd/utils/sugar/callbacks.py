"""Training-loop hooks that drive the EBOPs regulariser (reference src/hgq/utils/sugar/{ebops,beta_scheduler,
beta_pid}.py): they read the layers' ``_ebops`` counters and assign their ``_beta`` once per epoch.  The reference
classes are Keras callbacks; here ``Callback`` is the small protocol of the same method names, and ``fit`` below calls
it in Keras' order (train begin, then per epoch: begin, steps, end)."""

from __future__ import annotations

from collections.abc import Callable, Iterable, Sequence
from math import log10

import numpy as np
import torch

from ...layers.core.base import QLayerBase


class Callback:
    model = None

    def set_model(self, model):
        self.model = model

    def on_train_begin(self, logs=None):
        pass

    def on_epoch_begin(self, epoch, logs=None):
        pass

    def on_epoch_end(self, epoch, logs=None):
        pass


def _q_layers(model):
    return [m for m in model.modules() if isinstance(m, QLayerBase)]


def _top_layers(model):
    layers = getattr(model, 'layers', None)
    return list(layers) if layers is not None else [model]


def _counter(value) -> int:
    """A layer's ``ebops``: a python int (layers that add up their parts) or the uint32 variable."""
    if isinstance(value, torch.Tensor):
        return int(value.detach().cpu().view(torch.int32)) & 0xFFFFFFFF if value.dtype == torch.uint32 else int(value)
    return int(value)


def _assign_beta(model, beta: float):
    with torch.no_grad():
        for layer in model.modules():
            b = getattr(layer, '_beta', None)
            if isinstance(b, torch.Tensor):
                b.fill_(float(beta))


class FreeEBOPs(Callback):
    """Logs the sum of the layers' EBOPs counters at the end of every epoch (reference sugar/ebops.py:7-15)."""

    def on_epoch_end(self, epoch, logs=None):
        assert logs is not None
        logs['ebops'] = sum(_counter(layer._ebops) for layer in _q_layers(self.model) if layer.enable_ebops and layer._ebops is not None)


class BetaScheduler(Callback):
    """Sets every layer's beta to ``beta_fn(epoch)`` at the start of the epoch (reference sugar/beta_scheduler.py:9-31)."""

    def __init__(self, beta_fn: Callable[[int], float]):
        self.beta_fn = beta_fn

    def on_epoch_begin(self, epoch, logs=None):
        _assign_beta(self.model, self.beta_fn(epoch))

    def on_epoch_end(self, epoch, logs=None):
        assert isinstance(logs, dict)
        logs['beta'] = self.beta_fn(epoch)


class PieceWiseSchedule:
    """Beta interpolated between key points ``(epoch, beta, interp)``, ``interp`` in 'linear' / 'log' / 'constant' for
    the interval that starts at the point; constant after the last point (reference sugar/beta_scheduler.py:34-79)."""

    def __init__(self, intervals: Sequence[tuple[int, float, str]]):
        intervals = sorted(intervals, key=lambda v: v[0])
        self.epochs = [v[0] for v in intervals]
        self.betas = [v[1] for v in intervals]
        self.interpolations = [v[2] for v in intervals]
        assert all(interp in ('linear', 'log', 'constant') for interp in self.interpolations)

    def __call__(self, epoch):
        last = len(self.epochs) - 1
        idx0 = int(np.searchsorted(self.epochs, epoch, side='right')) - 1
        idx0, idx1 = max(0, min(idx0, last)), max(0, min(idx0 + 1, last))
        beta0, beta1 = self.betas[idx0], self.betas[idx1]
        epoch0, epoch1 = self.epochs[idx0], self.epochs[idx1]
        interp = self.interpolations[idx0]
        frac = (epoch - epoch0) / (epoch1 - epoch0 + 1e-9)
        if interp == 'linear':
            beta = beta0 + (beta1 - beta0) * frac
        elif interp == 'log':
            beta = beta0 * (beta1 / beta0) ** frac
        else:
            beta = beta0
        return float(beta)


class PID:
    """Discrete PID on the error ``sv - pv`` (``pv - sv`` with ``neg``); reference sugar/beta_pid.py:8-33."""

    def __init__(self, p: float, i: float, d: float, neg: bool):
        self.p, self.i, self.d, self.neg = p, i, d, neg
        self.integral = 0.0
        self.prev_error = 0.0

    def update_gains(self, p: float, i: float, d: float):
        self.p, self.i, self.d = p, i, d

    def update_gains_KcTiTd(self, Kp: float, Ti: float, Td: float):
        self.p, self.i, self.d = Kp, Kp / Ti, Kp * Td

    def __call__(self, sv: float, pv: float) -> float:
        err = sv - pv if not self.neg else pv - sv
        self.integral += err
        derivative = err - self.prev_error
        self.prev_error = err
        return self.p * err + self.i * self.integral + self.d * derivative


class BaseBetaPID(Callback):
    """Beta from a PID on the absolute EBOPs error (reference sugar/beta_pid.py:36-67)."""

    def __init__(self, target_ebops: float, p: float, i: float, d: float = 0.0) -> None:
        assert target_ebops > 0, 'Target EBOPs must be greater than 0.'
        self.pid = PID(p, i, d, neg=True)
        self.target_ebops = target_ebops

    def get_ebops(self) -> float:
        return float(sum(_counter(layer.ebops) for layer in _top_layers(self.model) if hasattr(layer, 'ebops')))

    def set_beta(self, beta: float):
        _assign_beta(self.model, beta)

    def on_epoch_begin(self, epoch, logs: dict | None = None):
        assert isinstance(logs, dict)
        ebops = self.get_ebops()
        beta = max(self.pid(self.target_ebops, ebops), 0.0)
        self.set_beta(beta)
        logs['beta'] = beta
        logs['ebops'] = ebops


class BetaPID(BaseBetaPID):
    """Steers beta so that the model's EBOPs reach ``target_ebops``: a PID on ``log10(ebops / target)`` producing
    ``log10(beta)`` (or on the ratio itself with ``log=False``), idle for ``warmup`` epochs, clamped to
    ``[min_beta, max_beta]``, damped by ``1 - damp_beta_on_target`` while below the target.  At the first controlled
    epoch the integral term is initialised so that the output equals the current beta (reference sugar/beta_pid.py:70-167)."""

    def __init__(self, target_ebops: float, init_beta: float | None = None, p: float = 1.0, i: float = 2e-3, d: float = 0.0,
                 warmup: int = 10, log: bool = True, max_beta: float = float('inf'), min_beta: float = 0.0,
                 damp_beta_on_target: float = 0.0) -> None:
        super().__init__(target_ebops, p, i, d)
        self.warmup, self.init_beta, self.log = warmup, init_beta, log
        self.max_beta, self.min_beta, self.damp_beta_on_target = max_beta, min_beta, damp_beta_on_target

    def get_avg_beta(self) -> float:
        betas = [float(layer._beta) for layer in self.model.modules() if isinstance(getattr(layer, '_beta', None), torch.Tensor)]
        return sum(betas) / len(betas) if betas else 0.0

    def on_train_begin(self, logs=None):
        if self.init_beta is not None:
            self.set_beta(self.init_beta)
        self.beta = self.get_avg_beta() if self.init_beta is None else self.init_beta
        self._ebops = self.get_ebops()

    def on_epoch_begin(self, epoch: int, logs: dict | None = None) -> None:
        assert isinstance(logs, dict)
        if epoch < self.warmup:
            if self.init_beta is not None:
                self.set_beta(self.init_beta)
            return
        ebops = self._ebops
        if epoch == self.warmup:
            # the integral term such that the controller's first output is the current beta: beta = p * P + i * I
            if not self.log:
                err = 1 - ebops / self.target_ebops
                self.pid.integral = (self.beta - self.pid.p * err) / self.pid.i - err
            else:
                err = log10(ebops / self.target_ebops + 1e-9)
                self.pid.integral = (log10(self.beta) - self.pid.p * err) / self.pid.i - err
        if self.log:
            beta = 10.0 ** self.pid(0, log10(ebops / self.target_ebops))
        else:
            beta = self.pid(1, ebops / self.target_ebops)
        if ebops < self.target_ebops:
            beta *= 1 - self.damp_beta_on_target
        beta = max(min(beta, self.max_beta), self.min_beta)
        self.set_beta(beta)
        self.beta = beta

    def on_epoch_end(self, epoch: int, logs: dict | None = None):
        assert isinstance(logs, dict)
        logs['beta'] = self.beta
        ebops = self.get_ebops()
        logs['ebops'] = ebops
        self._ebops = ebops


def fit(model, train_step: Callable, batches: Callable[[int], Iterable], epochs: int, callbacks: Sequence[Callback] = ()):
    """Minimal epoch loop in Keras' callback order.  ``batches(epoch)`` yields the arguments of ``train_step`` (which runs
    forward, backward and the optimizer and returns the loss); returns the per-epoch logs."""
    for cb in callbacks:
        cb.set_model(model)
    for cb in callbacks:
        cb.on_train_begin({})
    history = []
    for epoch in range(epochs):
        logs: dict = {}
        for cb in callbacks:
            cb.on_epoch_begin(epoch, logs)
        loss = None
        for batch in batches(epoch):
            loss = train_step(*batch) if isinstance(batch, (tuple, list)) else train_step(batch)
        if loss is not None:
            logs['loss'] = float(loss)
        for cb in callbacks:
            cb.on_epoch_end(epoch, logs)
        history.append(logs)
    return history
