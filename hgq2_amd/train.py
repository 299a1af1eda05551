"""Training-step plumbing for models built from the quantized layers: loss assembly, the SGD
update with the bit-width constraints folded in, and HIP-graph capture of a whole step.

What a Keras trainer does around the layers (reference call stack: tests/base.py:302-321):
sum the user loss, the ``add_loss`` terms (EBOPs * beta) and the variable regularizers; back-
propagate; ``w <- w - lr * g``; apply each variable's constraint.
"""

from __future__ import annotations

import operator

import torch

from . import ops
from .core import Layer, tree_cache
from .regularizers import MonoL1


class _SumLater(torch.autograd.Function):
    """The sum of one-element terms whose VALUE is written later (by the launch that joins the streams, or by the update);
    its gradient - the upstream gradient to every term - needs no value, so ``loss.backward()`` works on the result."""

    @staticmethod
    def forward(ctx, shape, *terms):
        ctx.shapes = [t.shape for t in terms]
        return terms[0].new_empty(shape)

    @staticmethod
    def backward(ctx, g):
        return (None,) + tuple(g.reshape(s) if ctx.needs_input_grad[1 + t] else None for t, s in enumerate(ctx.shapes))


def model_loss(model, base_loss, fold_regularizers: bool = False):
    """``base_loss + sum(add_loss terms) (+ variable regularizers)``.  With ``fold_regularizers``
    the MonoL1 terms are left out of the autograd graph: their constant gradient ``l1`` is added by
    :class:`SGD` inside the update kernel instead (same update, one launch less per variable)."""
    terms = [base_loss]
    cache = tree_cache(model) if isinstance(model, Layer) else None
    for m in (cache.layers if cache is not None else model.modules()):
        terms.extend(getattr(m, '_losses', ()))
    for p in (cache.regularised if cache is not None else model.parameters()):
        r = getattr(p, 'regularizer', None)
        if r is None or not p.requires_grad:  # Keras regularises trainable variables only
            continue
        if fold_regularizers and isinstance(r, MonoL1):
            continue
        terms.append(r(p))
    if ops._OVERLAP['depth'] and len(terms) > 1 and all(
            torch.is_tensor(t) and t.is_cuda and t.dtype == torch.float32 and t.numel() == 1 for t in terms):
        # inside `ops.overlap_ebops()` (EBOPs launches of this step may be running on the second stream): the total -
        # nothing but the caller's print-out reads it - is summed when the streams are joined for the last time, inside
        # the update's launch when :class:`SGD` makes it, and the backward pass starts from the terms themselves -
        # d total / d term = 1 - so the first stream does not wait for the second before the update
        total = _SumLater.apply(torch.broadcast_shapes(*[t.shape for t in terms]), *terms)
        held = list(terms)
        ops._OVERLAP['finish'].append((held, total.detach()))
        total._hgq_terms = [t for t in terms if t.requires_grad]
        return total
    ops.join_side()  # EBOPs terms issued on the second stream
    if len(terms) > 1 and all(torch.is_tensor(t) and t.is_cuda and t.dtype == torch.float32 and t.numel() == 1 for t in terms):
        # the same additions in the same order, one launch
        return ops.sum_scalars(terms).reshape(torch.broadcast_shapes(*[t.shape for t in terms]))
    loss = base_loss
    for term in terms[1:]:
        loss = loss + term
    return loss


class SGD:
    """Plain SGD (the optimizer of the reference's training test, tests/base.py:313) with the
    per-variable constraint applied after the update, as Keras optimizers do."""

    def __init__(self, params, lr: float = 0.01, fold_regularizers: bool = False):
        self.params = [p for p in params if p.requires_grad]
        self._owner_ids = frozenset(id(p) for p in self.params)  # the variables whose parked gradient pieces `step` consumes
        self.lr = float(lr)
        self.fold_regularizers = fold_regularizers
        self._unit = None

    def zero_grad(self, set_to_none: bool = True):
        for p in self.params:
            p._hgq_side = None
            if set_to_none:
                p.grad = None
            elif p.grad is not None:
                p.grad.zero_()

    def backward(self, loss):
        """``loss.backward()`` with the gradient sink of :class:`hgq2_amd.ops.side_gradients` open: the EBOPs terms leave
        their bit-width gradients on the variables as ``(upstream gradient, piece)`` pairs instead of sending them through
        autograd, and :meth:`step` adds the pieces inside the update kernel.  Same update as ``loss.backward()`` followed by
        :meth:`step`; about four launches fewer per quantized layer."""
        if loss.numel() != 1:
            raise ValueError('backward(loss) expects a scalar loss')
        if self._unit is None or self._unit.device != loss.device or self._unit.shape != loss.shape:
            self._unit = torch.ones_like(loss)  # the seed gradient: allocated once, also outside a captured graph
        terms = getattr(loss, '_hgq_terms', None)
        with ops.side_gradients(self._unit, self._owner_ids):
            if terms is not None:  # `model_loss` inside `ops.overlap_ebops()`: the sum is a plain value, its terms carry the graph
                torch.autograd.backward(terms, [self._unit.reshape(t.shape) for t in terms])
            else:
                loss.backward(self._unit)

    @torch.no_grad()
    def step(self):
        sums = ops.join_side(hand_over_sums=True)  # the loss terms' sum rides along with the update launch
        ws, gs, l1s, los, his, sides, post = [], [], [], [], [], [], []
        for p in self.params:
            side = list(getattr(p, '_hgq_side', None) or ())
            g = p.grad
            if g is None and not side:
                continue
            while len(side) > ops.SGD_SIDES:  # more pieces than the kernel takes: fold the surplus into one
                (s1, d1), (s2, d2) = side.pop(), side.pop()
                side.append((None, (d1 if s1 is None else s1 * d1) + (d2 if s2 is None else s2 * d2)))
            c = getattr(p, 'constraint', None)
            r = getattr(p, 'regularizer', None)
            bounds = c.bounds() if c is not None else (float('-inf'), float('inf'))
            if bounds is None:  # a constraint that is not a clip: applied after the update
                bounds = (float('-inf'), float('inf'))
                post.append((p, c))
            ws.append(p.data)
            gs.append(g)
            sides.append(side)
            l1s.append(r.l1 if (self.fold_regularizers and isinstance(r, MonoL1)) else 0.0)
            los.append(bounds[0])
            his.append(bounds[1])
        ride = sums.pop(0) if (ws and sums) else (None, None)
        for terms, out in sums:
            ops.sum_scalars_into(terms, out)
        if ws:
            ops.touch_state()  # written through `.data`: the version counters do not move
            ops.sgd_update_multi_(ws, gs, l1s, los, his, self.lr, sides, sum_terms=ride[0], sum_out=ride[1])
        for p, c in post:
            p.copy_(c(p))


class GraphedTrainStep:
    """One training step (forward, loss, backward, optimizer update) captured in a HIP graph.

    The step is launch-bound at the layer sizes this package targets (tens of small kernels), so
    the whole sequence is recorded once on a side stream and replayed; inputs are copied into
    static buffers before each replay.  ``loss_fn(outputs, labels)`` must be built from capturable
    operations (``hgq2_amd.ops.sparse_ce`` is)."""

    def __init__(self, model, loss_fn, optimizer: SGD, example_x, example_y, warmup: int = 3, overlap: bool = True,
                 warmup_data=None, feed: 'ResidentBatches | None' = None):
        """The recording is preceded by ``warmup`` real training steps on the example batch (operators create their
        per-stream scratch there, not inside the graph) - or, with ``warmup_data`` (a sequence of ``(x, y)`` of the
        example's shapes), by one step on each of those: a loop that counts its steps hands over its first batches and
        starts replaying with the next one; their losses are left in ``warmup_losses``.

        ``feed``: the step draws its batch itself (:class:`ResidentBatches`: a launch at the head of the recorded step
        that reads the next rows of a data set in device memory) and adds its loss to ``total``; ``step()`` without
        arguments is then a replay and nothing else.  The ``warmup`` steps draw the feed's first batches."""
        self.model, self.loss_fn, self.opt = model, loss_fn, optimizer
        self.overlap = overlap  # EBOPs launches and the loss sum on a second branch of the graph, beside loss and backward
        self.feed = feed
        self.x = example_x.clone()
        self.y = example_y.clone()
        self.total = torch.zeros((), dtype=torch.float32, device=example_x.device)  # with a feed: the sum of the steps' losses
        self.loss = None
        self.warmup_losses = []
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            if feed is not None:
                for _ in range(warmup):
                    self.warmup_losses.append(self._step().clone())
            elif warmup_data is None:
                for _ in range(warmup):
                    self._step()
            else:
                if len(warmup_data) < 1:
                    raise ValueError('the recording needs at least one step before it')
                for wx, wy in warmup_data:
                    self.x.copy_(wx), self.y.copy_(wy)
                    self.warmup_losses.append(self._step().clone())
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.opt.zero_grad(set_to_none=True)
        self.graph = torch.cuda.CUDAGraph()
        # captured on the stream the warm-up ran on: scratch that operators keep per stream (allocated and cleared once,
        # during the warm-up) is found again instead of being created, and cleared, inside the graph
        with torch.cuda.graph(self.graph, stream=side):
            self.loss = self._step()

    def _step(self):
        import contextlib

        if self.feed is not None:
            self.feed.draw(self.x, self.y)
        with ops.overlap_ebops() if self.overlap else contextlib.nullcontext():
            self.opt.zero_grad(set_to_none=True)
            out = self.model(self.x, training=True)
            loss = model_loss(self.model, self.loss_fn(out, self.y), self.opt.fold_regularizers)
            self.opt.backward(loss)
            self.opt.step()
        loss = loss.detach()
        if self.feed is not None:
            self.total.add_(loss.reshape(()))
        return loss

    def __call__(self, x=None, y=None):
        if x is not None:
            self.x.copy_(x)
        if y is not None:
            self.y.copy_(y)
        ops.touch_state()  # the replayed kernels update the variables
        self.graph.replay()
        return self.loss

    def eager(self, x, y):
        """The same step launched kernel by kernel on a batch of another size (the last, shorter batch of an epoch)."""
        keep = self.x, self.y, self.feed
        self.x, self.y, self.feed = x, y, None
        try:
            return self._step()
        finally:
            self.x, self.y, self.feed = keep


class ResidentBatches:
    """The batches of an epoch loop over a data set that lives in device memory, drawn by a launch of their own
    (``hgq_gather_batch``) so that a recorded step can fetch its batch when it is replayed: ``start_epoch(order)`` lays
    down the epoch's order (a permutation of the rows, or ``None`` for the rows as they stand) and rewinds; every
    ``draw(x_buf, y_buf)`` - eager or replayed - fills the buffers with the next ``x_buf.shape[0]`` rows of that order."""

    def __init__(self, x, y):
        if x.shape[0] != y.shape[0] or x.shape[0] < 1:
            raise ValueError('x and y must hold the same, non-zero number of samples')
        self.x, self.y = x.contiguous(), y.contiguous()
        n = x.shape[0]
        self._identity = torch.arange(n, dtype=torch.int64, device=x.device)
        self.order = self._identity.clone()
        self.state = torch.zeros(2, dtype=torch.int64, device=x.device)

    @staticmethod
    def covers(x, y) -> bool:
        """Rows of whole 32-bit words on the GPU."""
        return all(t.is_cuda and t.dim() >= 1 and t.shape[0] >= 1 and (t[0].numel() * t.element_size()) % 4 == 0 and t[0].numel() > 0
                   for t in (x, y))

    def start_epoch(self, order=None):
        self.order.copy_(self._identity if order is None else order)
        self.state.zero_()

    def draw(self, x_buf, y_buf):
        ops.gather_batch(self.x, self.y, self.order, self.state, x_buf, y_buf)


_version_of = operator.attrgetter('_version')


def _raw_stream(device_index: int) -> int:
    """The current HIP stream of the device as an integer handle (the short way when this torch has it)."""
    get = getattr(torch._C, '_cuda_getCurrentRawStream', None)
    return get(device_index) if get is not None else torch.cuda.current_stream(device_index).cuda_stream


class FusedQDenseStack:
    """One SGD training step of a stack of :class:`QDense` layers with mean sparse categorical
    cross-entropy, executed by the whole-step kernels (two launches once the quantized weight image of
    the previous step can be reused, see ``hgq_mlp_train_step_cached``).

    It updates exactly the variables the layer-by-layer path updates (kernels, biases, every
    bit-width variable, the tracked integer bits, ``ebops``) with the same arithmetic; it exists
    because at these layer sizes a step made of per-layer launches is bound by launch latency.
    Requirements (checked): 2-D inputs, widths up to 64, plain KIF/WRAP input quantizers with
    batch-shared bit-widths, plain KBI SAT / SAT_SYM kernel and bias quantizers, relu or linear
    activations, no kernel / bias regularizers or constraints, MonoL1 or no regularizer and clip
    constraints on the bit-widths.
    """

    def __init__(self, layers, lr: float = 0.01):
        import ctypes

        from . import _lib
        from .layers import QDense
        from .quantizer.internal import FixedPointQuantizerKBI, FixedPointQuantizerKIF
        from .regularizers import MonoL1 as _L1

        layers = list(getattr(layers, 'layers', layers))
        if not layers or not all(isinstance(layer, QDense) and layer.built for layer in layers):
            raise ValueError('FusedQDenseStack needs a non-empty sequence of built QDense layers')
        self.layers, self.lr = layers, float(lr)
        self._lib, self._ct = _lib, ctypes
        arr = (_lib.MlpLayer * len(layers))()
        inf = float('inf')

        def var_params(p):
            r, c = getattr(p, 'regularizer', None), getattr(p, 'constraint', None)
            if r is not None and not isinstance(r, _L1):
                raise ValueError('only MonoL1 regularizers can be folded into the fused update')
            b = c.bounds() if c is not None else (-inf, inf)
            if b is None:
                raise ValueError('only clip-type constraints can be folded into the fused update')
            return (r.l1 if (r is not None and p.requires_grad) else 0.0), b[0], b[1]

        ptr = lambda t: t.data_ptr() if t is not None else None  # noqa: E731
        for n, layer in enumerate(layers):
            qi = layer.iq.quantizer if layer.enable_iq else None
            qk, qb = layer.kq.quantizer, (layer.bq.quantizer if layer.bq is not None else None)
            ok = (qi is not None and layer.iq.plain and isinstance(qi, FixedPointQuantizerKIF) and qi.overflow_mode == 'WRAP'
                  and qi.trainable and tuple(qi._i.shape) == (1, layer._kernel.shape[0])
                  and layer.kq.plain and isinstance(qk, FixedPointQuantizerKBI) and qk.overflow_mode != 'WRAP'
                  and (qb is None or (layer.bq.plain and isinstance(qb, FixedPointQuantizerKBI) and qb.overflow_mode != 'WRAP'))
                  and layer._act_name in ('relu', 'linear') and not layer.enable_oq
                  and not any(q is not None and q.stochastic for q in (qi, qk, qb))
                  and all(getattr(p, 'regularizer', None) is None and getattr(p, 'constraint', None) is None
                          for p in (layer._kernel, layer.bias) if p is not None))
            if not ok:
                raise ValueError(f'layer {n} ({layer.name}) is outside what the fused QDense step covers')
            it = arr[n]
            it.K, it.N = layer._kernel.shape
            it.act = _lib.ACT_RELU if layer._act_name == 'relu' else _lib.ACT_NONE
            km = lambda q: q._mode(True) | _lib.MODE_K_U8  # noqa: E731  (`_k` variables are uint8)
            it.mode_in, it.mode_ker, it.mode_bias = km(qi), km(qk), (km(qb) if qb is not None else 0)
            it.w, it.bias = ptr(layer._kernel), ptr(layer.bias)
            it.k_in, it.i_in, it.f_in = ptr(qi._k), ptr(qi._i), ptr(qi._f)
            it.k_ker, it.b_ker, it.i_ker = ptr(qk._k), ptr(qk._b), ptr(qk._i)
            if qb is not None:
                it.k_bias, it.b_bias, it.i_bias = ptr(qb._k), ptr(qb._b), ptr(qb._i)
            it.decay = qi._decay_host
            if layer.enable_ebops:
                it.beta, it.ebops = ptr(layer._beta), ptr(layer._ebops)
            it.par_factor, it.n_parallel = float(layer.parallelization_factor), float(layer.n_parallel)
            it.ebops_factor = float(layer.ebops_factor)
            it.bias_size = float(layer.units)
            it.f_in_l1, it.f_in_lo, it.f_in_hi = var_params(qi._f)
            it.b_ker_l1, it.b_ker_lo, it.b_ker_hi = var_params(qk._b)
            it.i_ker_l1, it.i_ker_lo, it.i_ker_hi = var_params(qk._i)
            it.train_i_ker = int(qk._i.requires_grad)
            if qb is not None:
                it.b_bias_l1, it.b_bias_lo, it.b_bias_hi = var_params(qb._b)
                it.i_bias_l1, it.i_bias_lo, it.i_bias_hi = var_params(qb._i)
                it.train_i_bias = int(qb._i.requires_grad)
        self._arr = arr
        self._ws = None
        # every variable the step reads: an in-place change from outside (seen through the tensors'
        # version counters, which the kernels do not touch) invalidates the cached weight image
        self._vars = [t for layer in layers for t in self._layer_vars(layer)]
        self._versions = None
        self.device = layers[0]._kernel.device
        self.loss = torch.zeros((), dtype=torch.float32, device=self.device)
        self._loss_ptr, self._ws_ptr = self.loss.data_ptr(), None
        self._dev_index = self.device.index if self.device.index is not None else torch.cuda.current_device()
        self._K0 = int(arr[0].K)
        self._need = {}  # rows -> workspace floats
        self._decay_of = [(it, layer.iq.quantizer) for it, layer in zip(arr, layers)]

    def invalidate(self):
        """Forget the cached quantized-weight image (after writing the variables in a way neither version counters nor
        this package's own updaters see, e.g. through a raw pointer)."""
        self._versions = None

    @staticmethod
    def _layer_vars(layer):
        qs = [layer.iq.quantizer, layer.kq.quantizer] + ([layer.bq.quantizer] if layer.bq is not None else [])
        out = [layer._kernel] + ([layer.bias] if layer.bias is not None else [])
        for q in qs:
            out += [v for v in (getattr(q, '_k', None), getattr(q, '_i', None), getattr(q, '_f', None), getattr(q, '_b', None)) if v is not None]
        return out

    def step(self, x, labels):
        """Run one training step in place; returns the loss tensor (cross-entropy + sum of EBOPs * beta
        + MonoL1 regularisation terms, i.e. the full training loss)."""
        if not (x.is_cuda and x.dtype == torch.float32 and x.is_contiguous() and x.dim() == 2 and x.shape[1] == self._K0):
            raise ValueError('x must be a contiguous float32 GPU tensor [rows, K]')
        rows = x.shape[0]
        if not (labels.is_cuda and labels.dtype == torch.int64 and labels.is_contiguous() and labels.shape == (rows,)):
            raise ValueError('labels must be a contiguous int64 GPU tensor [rows]')
        # (the host side of a step is a few microseconds of Python around one foreign call: at 16384 rows the two
        # launches take the GPU about 30 us, so what is looked up per step is kept to what can change between steps)
        lib = self._lib.load()
        need = self._need.get(rows)
        if need is None:
            need = lib.hgq_mlp_workspace(self._arr, len(self.layers), rows)
            if need < 0:
                self._lib.check(-3, 'hgq_mlp_workspace')
            self._need[rows] = need
        for it, q in self._decay_of:
            it.decay = q._decay_host  # follows the variable
        # the kernels of this class do not move version counters or the state epoch: both unchanged = nobody else wrote
        versions = (*map(_version_of, self._vars), ops.STATE_EPOCH[0])
        current = self._versions == versions
        if self._ws is None or self._ws.numel() < need:
            self._ws = torch.empty(need, dtype=torch.float32, device=self.device)
            self._ws_ptr, current = self._ws.data_ptr(), False
        rc = lib.hgq_mlp_train_step_cached(self._arr, len(self.layers), x.data_ptr(), labels.data_ptr(), rows, self.lr, self._loss_ptr,
                                           self._ws_ptr, int(current), _raw_stream(self._dev_index))
        if rc:
            self._lib.check(rc, 'hgq_mlp_train_step_cached')
        self._versions = versions
        return self.loss


class _FusedStep:
    """The whole-step kernels behind the call signature of :class:`GraphedTrainStep`."""

    path = 'fused'

    def __init__(self, stack: FusedQDenseStack):
        self.stack = stack

    def __call__(self, x, y):
        return self.stack.step(x, y)


def train_step_for(model, example_x, example_y, lr: float = 0.01, loss: str = 'sparse_ce', fused: bool | None = None,
                   warmup_data=None, feed=None, warmup: int = 3):
    """A callable ``step(x, y) -> loss`` that runs one SGD training step of ``model`` on the fastest path that covers it.

    A built stack of :class:`QDense` layers trained with mean sparse categorical cross-entropy and within what
    :class:`FusedQDenseStack` checks (widths up to 64, the default quantizer kinds, an LDS plan that fits) runs on the
    whole-step kernels; every other model, and ``loss='mse'``, runs the per-layer operators replayed from a HIP graph
    (:class:`GraphedTrainStep` with :class:`SGD`, regularizers folded into the update).  Both paths update the same
    variables with the same arithmetic (the whole-step kernels restate the per-layer sequence), so the choice changes
    the time per step and nothing else.  ``fused=False`` forces the per-layer path, ``fused=True`` raises where the
    whole-step path does not apply.  The returned object's ``path`` is ``'fused'`` or ``'layers_graph'``.
    ``warmup_data``, ``feed``, ``warmup``: see :class:`GraphedTrainStep` (the whole-step path needs no steps before it and
    takes none: ``warmup_losses`` is then empty; it does not use a ``feed`` either)."""
    if loss not in ('sparse_ce', 'mse'):
        raise ValueError(f"loss must be 'sparse_ce' or 'mse', got {loss!r}")
    if not model.built:
        model(example_x, training=False)  # creates the variables; an inference call leaves the integer-bit trackers alone
    if fused is not False and loss == 'sparse_ce':
        try:
            stack = FusedQDenseStack(model, lr=lr)
            if example_x.dim() != 2 or example_x.shape[1] != stack._arr[0].K:
                raise ValueError('the fused QDense step takes [rows, features] inputs')
            from . import _lib

            lib = _lib.load()
            if lib.hgq_mlp_workspace(stack._arr, len(stack.layers), example_x.shape[0]) < 0:
                raise ValueError('the fused QDense step does not cover this stack: ' + (lib.hgq_last_error() or b'').decode())
            return _FusedStep(stack)
        except ValueError:
            if fused:
                raise
    elif fused:
        raise ValueError('the fused QDense step computes sparse categorical cross-entropy only')
    loss_fn = ops.sparse_ce if loss == 'sparse_ce' else ops.mse
    step = GraphedTrainStep(model, loss_fn, SGD(model.parameters(), lr=lr, fold_regularizers=True), example_x, example_y,
                            warmup=warmup, warmup_data=warmup_data, feed=feed)
    step.path = 'layers_graph'
    return step


def folded_regularizer_loss(model) -> float:
    """Sum of the MonoL1 terms that :func:`model_loss` leaves out with ``fold_regularizers`` (trainable variables only)."""
    total = 0.0
    with torch.no_grad():
        for p in model.parameters():
            r = getattr(p, 'regularizer', None)
            if isinstance(r, MonoL1) and p.requires_grad:
                total += float(r(p))
    return total


def fit(model, x, y, *, loss: str = 'sparse_ce', lr: float = 0.01, batch_size: int = 1024, epochs: int = 1, callbacks=(),
        shuffle: bool = True, seed: int | None = None, fused: bool | None = None):
    """Train ``model`` on the resident tensors ``x`` / ``y`` (first axis: samples) with plain SGD, the way the reference's
    users call ``model.fit`` (reference tests/base.py:313-331; the epoch hooks of src/hgq/utils/sugar/ drive beta from it):
    per epoch the callbacks' ``on_epoch_begin``, the batches in order (shuffled anew per epoch with ``shuffle``; the last
    one may be shorter), ``on_epoch_end`` with ``logs['loss']`` = the mean of the epoch's step losses.  Returns the list
    of the epochs' logs.

    The steps run on the fastest path that covers the model (:func:`train_step_for`): full batches through the
    whole-step kernels or a HIP-graph replay - the recording's preparatory steps are the loop's own first batches, so
    every batch is trained on exactly once - and a shorter last batch through the same kernels launched one by one.
    On the replayed path the recorded step fetches its own batch (:class:`ResidentBatches`: the epoch's order lies in
    device memory and a launch at the head of the step gathers the next rows) and adds its loss to a running sum, so a
    step costs the host one replay call.  The epoch's loss is summed on the device and read once per epoch.  On the per-layer path the MonoL1 terms of the
    variables are applied inside the update launch and are not part of a step's loss value: their sum
    (:func:`folded_regularizer_loss`, of the order of 1e-4 with the default 1e-8 factors) is added to ``logs['loss']``
    once, from the variables as they stand when the epoch ends; the whole-step kernels include it in every step."""
    n = int(x.shape[0])
    if n < 1 or int(y.shape[0]) != n:
        raise ValueError('x and y must hold the same, non-zero number of samples')
    if not x.is_cuda:
        raise ValueError('fit trains on GPU tensors: the product has no CPU path')
    batch_size = min(int(batch_size), n)
    n_full, tail = divmod(n, batch_size)
    gen = torch.Generator(device='cpu')
    if seed is not None:
        gen.manual_seed(int(seed))
    for cb in callbacks:
        cb.set_model(model)
    for cb in callbacks:
        cb.on_train_begin({})
    step = None
    history = []
    # a data set of whole 32-bit words per row is fed by a launch inside the recorded step (no copies between replays)
    feed = ResidentBatches(x, y) if (fused is not True and ResidentBatches.covers(x, y)) else None
    for epoch in range(epochs):
        logs: dict = {}
        for cb in callbacks:
            cb.on_epoch_begin(epoch, logs)
        order = torch.randperm(n, generator=gen).to(x.device) if shuffle else None

        def batch(b, size=batch_size):
            lo = b * batch_size
            if order is None:
                return x[lo:lo + size], y[lo:lo + size]
            idx = order[lo:lo + size]
            return x.index_select(0, idx), y.index_select(0, idx)

        total = torch.zeros((), dtype=torch.float32, device=x.device)
        first = 0
        if feed is not None:
            feed.start_epoch(order)
        if step is None:
            # the steps before the recording are this epoch's first batches
            warm = [batch(b) for b in range(min(3, n_full))]
            step = train_step_for(model, *warm[0], lr=lr, loss=loss, fused=fused, warmup_data=warm, feed=feed, warmup=len(warm))
            if isinstance(step, _FusedStep):
                feed = None  # the whole-step kernels read the batch where it lies
            done = getattr(step, 'warmup_losses', [])
            for l in done:
                total += l.reshape(())
            first = len(done)
        if feed is not None:
            step.total.zero_()
            for b in range(first, n_full):
                step()
            total += step.total
        else:
            for b in range(first, n_full):
                total += step(*batch(b)).reshape(())
        if tail:
            bx, by = batch(n_full, tail)
            if isinstance(step, _FusedStep):
                total += step(bx.contiguous(), by.contiguous()).reshape(())
            else:
                total += step.eager(bx, by).reshape(())
        logs['loss'] = float(total) / (n_full + (1 if tail else 0))
        if not isinstance(step, _FusedStep):
            logs['loss'] += folded_regularizer_loss(model)
        for cb in callbacks:
            cb.on_epoch_end(epoch, logs)
        history.append(logs)
    return history

