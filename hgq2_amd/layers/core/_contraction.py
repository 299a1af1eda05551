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


def dense_contraction(x, iq, qkernel2d, qbias1d, act_name, training):
    """x [..., K] -> [..., N].  Returns the 2-D result [rows, N]."""
    K, N = qkernel2d.shape
    x2d = x.reshape(-1, K)
    if not x2d.is_contiguous():
        x2d = x2d.contiguous()
    act_code = _lib.ACT_RELU if act_name == 'relu' else _lib.ACT_NONE
    bw_rows = fused_iq_rows(iq, tuple(x.shape), K, training)
    fused_bwd = K <= ops.FUSED_BWD_MAX and N <= ops.FUSED_BWD_MAX
    if bw_rows and fused_bwd:
        q = iq.quantizer
        y, amax = ops.qdense(x2d, q._k.view(-1), q._i.view(-1), q._f.view(-1), qkernel2d, qbias1d, act_code,
                             q._mode(True), bw_rows, True)
        q._track(amax, True)
        return y, act_code != _lib.ACT_NONE
    if iq is not None:
        x2d = iq(x, training=training).reshape(-1, K)
        if not x2d.is_contiguous():
            x2d = x2d.contiguous()
    if fused_bwd:
        y, _ = ops.qdense(x2d, None, None, None, qkernel2d, qbias1d, act_code, 0, 0, False)
        return y, act_code != _lib.ACT_NONE
    # shapes beyond the fused backward kernel: plain library GEMM on the quantized operands
    y = x2d @ qkernel2d
    if qbias1d is not None:
        y = y + qbias1d
    return y, False


def dense_ebops_fast(iq, kq, bq, K, N, scale, bias_size):
    """EBOPs through the fused kernel when the quantizers are the fixed-point kinds it covers.
    Returns ``(ebops, uint32 bit pattern)`` or ``None`` when the generic path must be used."""
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
    return ops.dense_ebops(
        qi._k.view(-1), qi._i.view(-1), qi._third().view(-1), qk._k.view(-1), qk._b.view(-1),
        qb._k.view(-1) if qb is not None else None, qb._b.view(-1) if qb is not None else None, P, K, N, scale,
        bias_size, qi._mode(True), qk._mode(True), qb._mode(True) if qb is not None else 0)
