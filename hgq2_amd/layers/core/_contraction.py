"""Shared implementation of the dense contraction ``act(q_in(x) @ q_w(W) + q_b(b))`` used by
QDense and by QEinsumDense equations that reshape to a GEMM."""

from __future__ import annotations

import torch

from ... import _lib, ops
from ...quantizer.internal import FixedPointQuantizerKBI, FixedPointQuantizerKIF
from ...quantizer.internal.base import bw_layout

_ACTIVATIONS = {
    None: None,
    'linear': None,
    'relu': torch.relu,
    'sigmoid': torch.sigmoid,
    'tanh': torch.tanh,
    'softplus': torch.nn.functional.softplus,
    'gelu': torch.nn.functional.gelu,
    'elu': torch.nn.functional.elu,
}


def get_activation(act):
    if callable(act):
        return act, getattr(act, '__name__', 'custom')
    if act in _ACTIVATIONS:
        return _ACTIVATIONS[act], act or 'linear'
    raise ValueError(f'unknown activation {act!r}')


def fused_iq_rows(iq, x_shape, K, training):
    """``bw_rows`` if the input quantizer can be fused into the GEMM operand load, else 0.

    Fusable: a plain (no scaler / noise / affine) KIF quantizer on its WRAP training branch whose
    bit-widths form a [bw_rows, K] table over the trailing axes of the input."""
    if iq is None or not iq.plain:
        return 0
    q = iq.quantizer
    if not isinstance(q, FixedPointQuantizerKIF) or not q.wrap_training_fusable(training):
        return 0
    layout = bw_layout(q._i.shape, x_shape)
    if layout is None or layout[1] != 1 or layout[0] % K != 0 or not _covers_trailing(q._i.shape, K):
        return 0
    return layout[0] // K


def _covers_trailing(bw_shape, K):
    """The bit-width tensor is fully heterogeneous over the trailing axes that make up K."""
    suffix = 1
    for s in reversed(tuple(bw_shape)):
        suffix *= s
        if suffix == K:
            return True
        if suffix > K:
            return False
    return False


class DeferredTracking:
    """Abs-max slices of a fused input quantizer whose integer-bit update has not run yet."""

    def __init__(self, quantizer, amax):
        self.quantizer, self.amax = quantizer, amax

    def flush(self):
        if self.amax is not None:
            self.quantizer._track(self.amax, True)
            self.amax = None


FUSED_TRACK_MAX = 65536  # slices * entries the single-workgroup EBOPs kernel is allowed to walk


def dense_contraction(x, iq, qkernel2d, qbias1d, act_name, training, oq=None, out_shape=None):
    """x [..., K] -> [rows, N].  Returns ``(y, activation applied, DeferredTracking or None, output quantizer applied)``.

    ``oq`` / ``out_shape``: the layer's output quantizer and the shape it sees.  When it is of the kind the input
    quantizer fusion takes (plain KIF on its WRAP training branch, a table over the trailing axes) and nothing but a relu
    stands between the contraction and it, the contraction kernel applies it to the tile it stores and leaves its abs-max
    trackers as slices; its integer bits are then updated here as its own call would."""
    K, N = qkernel2d.shape
    x2d = x.reshape(-1, K)
    if not x2d.is_contiguous():
        x2d = x2d.contiguous()
    act_code = _lib.ACT_RELU if act_name == 'relu' else _lib.ACT_NONE
    bw_rows = fused_iq_rows(iq, tuple(x.shape), K, training)
    fused_bwd = K <= ops.FUSED_BWD_MAX and N <= ops.FUSED_BWD_MAX
    if bw_rows and fused_bwd:
        q = iq.quantizer
        po = 0
        if oq is not None and out_shape is not None and act_name in (None, 'linear', 'relu'):
            po = fused_iq_rows(oq, tuple(out_shape), N, training)
        if po and _lib.load().hgq_qdense_fwd_oq_supported(x2d.shape[0], K, N, bw_rows, po, q._mode(True), oq.quantizer._mode(True)):
            qo = oq.quantizer
            yq, amax, oamax = ops.qdense_oq(x2d, q._k.view(-1), q._f.view(-1), qkernel2d, qbias1d, qo._k.view(-1), qo._i.view(-1),
                                            qo._f.view(-1), act_code, q._mode(True), qo._mode(True), bw_rows, po)
            qo._track(oamax, True)
            return yq, act_code != _lib.ACT_NONE, DeferredTracking(q, amax), True
        y, amax = ops.qdense(x2d, q._k.view(-1), q._i.view(-1), q._f.view(-1), qkernel2d, qbias1d, act_code,
                             q._mode(True), bw_rows, True)
        return y, act_code != _lib.ACT_NONE, DeferredTracking(q, amax), False
    if iq is not None:
        x2d = iq(x, training=training).reshape(-1, K)
        if not x2d.is_contiguous():
            x2d = x2d.contiguous()
    if fused_bwd:
        y, _ = ops.qdense(x2d, None, None, None, qkernel2d, qbias1d, act_code, 0, 0, False)
        return y, act_code != _lib.ACT_NONE, None, False
    # shapes beyond the fused backward kernel: the implicit-GEMM kernels in their 1 x 1 form
    y = ops.matmul_bias_act(x2d, qkernel2d, qbias1d, act_code)
    return y, act_code != _lib.ACT_NONE, None, False


def dense_contraction_mean(x, iq, qkernel2d, qbias1d, act_name, training, mean_rows):
    """``dense_contraction`` followed by a mean over groups of ``mean_rows`` consecutive rows, as one launch each way: returns
    ``(means [rows / mean_rows, N], DeferredTracking or None)``, or ``None`` where the kernels do not cover the case (the caller
    then contracts and averages in two steps).  The contraction's own output never leaves the operator."""
    K, N = qkernel2d.shape
    if act_name not in (None, 'linear', 'relu') or not x.is_cuda or x.numel() == 0:
        return None
    bw_rows = fused_iq_rows(iq, tuple(x.shape), K, training) if iq is not None else 0
    if iq is not None and not bw_rows:
        return None  # the quantizer runs as a launch of its own
    q = iq.quantizer if bw_rows else None
    mode = q._mode(True) if q is not None else 0
    x2d = x.reshape(-1, K)
    if not x2d.is_contiguous():
        x2d = x2d.contiguous()
    if not ops.qdense_mean_supported(x2d.shape[0], K, N, bw_rows, mean_rows, mode):
        return None
    act_code = _lib.ACT_RELU if act_name == 'relu' else _lib.ACT_NONE
    ymean, amax = ops.qdense_mean(x2d, q._k.view(-1) if q is not None else None, q._f.view(-1) if q is not None else None, qkernel2d,
                                  qbias1d, act_code, mode, bw_rows, mean_rows)
    return ymean, (DeferredTracking(q, amax) if q is not None else None)


def dense_ebops_term(layer, iq, kq, bq, K, N, bias_size, deferred):
    """``ebops * beta`` through the fused kernel (which also assigns the layer's ``_ebops`` and, when
    ``deferred`` tracking is pending and small enough, updates the input quantizer's ``_i`` first).
    Returns ``None`` when the quantizers are not the fixed-point kinds the kernel covers."""
    qi, qk = iq.quantizer, kq.quantizer
    if not isinstance(qi, (FixedPointQuantizerKIF, FixedPointQuantizerKBI)) or not isinstance(qk, FixedPointQuantizerKBI):
        return None
    qb = bq.quantizer if bq is not None else None
    if qb is not None and not isinstance(qb, FixedPointQuantizerKBI):
        return None
    if not _covers_trailing(qi._i.shape, K) or qi._i.numel() % K != 0 or K > 4096 or qk._b.numel() != K * N:
        return None
    if qb is not None and qb._b.numel() != N:
        return None
    P = qi._i.numel() // K
    amax = None
    if deferred is not None and deferred.amax is not None:
        if deferred.quantizer is qi and deferred.amax.numel() <= FUSED_TRACK_MAX:
            amax, deferred.amax = deferred.amax, None
        else:
            deferred.flush()
    decay = qi._decay_host if amax is not None else 0.0
    _, term = ops.dense_ebops(
        qi._k.view(-1), qi._i.view(-1), qi._third().view(-1), qk._k.view(-1), qk._b.view(-1),
        qb._k.view(-1) if qb is not None else None, qb._b.view(-1) if qb is not None else None, P, K, N,
        layer.parallelization_factor, layer.n_parallel, layer.ebops_factor, bias_size, qi._mode(True), qk._mode(True), qb._mode(True) if qb is not None else 0,
        amax=amax, decay=decay, beta=layer._beta, ebops_var=layer._ebops.view(torch.int32),
        owners=(qi._i, qi._third(), qk._b, qb._b if qb is not None else None))
    return term
