"""GPU parity at the full sizes of the benchmark configurations, and of the seams and branches the smaller tests do
not reach: the standalone quantizer at 4 Mi elements, the stateless callable driven the way the reference drives it,
the KBI WRAP state machine (training and calibration) with batch-shared bit-widths, the ``Quantizer`` wrapper with
scaler / noise blend / affine map, and the backward pass of the per-particle and image configurations.

Bars: quantized values, tracked integer bits, keep-negative flags and EBOPs bit-exact; everything that is a sum in
fp32 within 1e-5 of the sum of the absolute values of its terms (the oracle evaluates its contractions in float64 for
these tests, ``oracle.hgq_ref.ACC64``, so the bound measures the kernel and not the oracle's own summation order)."""

import math

import numpy as np
import pytest
import torch

from oracle import fixed_point as ofp
from oracle import hgq_ref as ref
from oracle import twin

pytestmark = pytest.mark.gpu
RTOL = 1e-5


def _close_scaled(got, want, scale, what, rtol=RTOL):
    got, want, scale = got.detach().double().cpu(), want.detach().double(), scale.detach().double()
    err = (got.reshape(want.shape) - want).abs()
    tol = rtol * scale.reshape(want.shape) + 1e-30
    ratio = (err / tol).reshape(-1)
    at = int(ratio.argmax())
    assert float(ratio[at]) <= 1.0, (f'{what}: error is {float(ratio[at]):.2f} x the bound at element {at}: got '
                                     f'{float(got.reshape(-1)[at]):.6e}, want {float(want.reshape(-1)[at]):.6e}, sum of |terms| '
                                     f'{float(scale.reshape(-1)[at]):.3e} (max err anywhere {float(err.max()):.3e})')


def _close_tensor(got, want, what, rtol=RTOL):
    """Per element within rtol * (|want| + max|want|): for gradients that are not a plain sum of products."""
    want = want.detach().double()
    _close_scaled(got, want, want.abs() + want.abs().max() + 1e-12, what, rtol)


# --------------------------------------------------------------------------------------------------------------
# configuration 1: the standalone quantizer at its full size
# --------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize('overflow_mode', ['WRAP', 'SAT', 'SAT_SYM'])
@pytest.mark.parametrize('training', [True, False])
def test_standalone_quantizer_at_4Mi(dev, overflow_mode, training):
    """4 Mi fp32 elements, x ~ N(0, 4), per-element k = 1, i ~ U{0..4}, f ~ U{0..8}, RND: values bit-exact in
    training and inference mode, dx / di / df (training) within 1e-5 per element (no sums are involved)."""
    from hgq2_amd import _lib, ops

    n = 4 * 1024 * 1024
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(n, generator=g) * 2.0).requires_grad_(training)
    k = torch.ones(n)
    i = torch.randint(0, 5, (n,), generator=g).float().requires_grad_(training)
    f = torch.randint(0, 9, (n,), generator=g).float().requires_grad_(training)
    gy = torch.randn(n, generator=g)
    q = ofp.get_fixed_quantizer('RND', overflow_mode)
    want = q(x, k, i, f, training, None)
    if not training:
        want = torch.where(k + i + f > 0, want, torch.zeros_like(want))
    mode = _lib.mode_bits('RND', overflow_mode, training=training)
    xd, idv, fd = (t.detach().to(dev).requires_grad_(training) for t in (x, i, f))
    y, _, _ = ops.quantize(xd, k.to(dev), idv, fd, mode)
    assert torch.equal(y.detach().cpu(), want.detach())
    if not training:
        return
    want.backward(gy)
    y.backward(gy.to(dev))
    for got, ref_g, name in ((xd.grad, x.grad, 'dx'), (idv.grad, i.grad, 'di'), (fd.grad, f.grad, 'df')):
        ref_g = torch.zeros(n) if ref_g is None else ref_g
        got = torch.zeros(n) if got is None else got.cpu()
        np.testing.assert_allclose(got.numpy(), ref_g.numpy(), rtol=RTOL, atol=1e-30, err_msg=f'{overflow_mode} {name}')


@pytest.mark.parametrize('overflow_mode', ['WRAP', 'SAT', 'SAT_SYM'])
@pytest.mark.parametrize('kbi', [False, True])
def test_standalone_quantizer_fwd_bwd_in_one_launch_at_4Mi(dev, overflow_mode, kbi):
    """``hgq_quantize_fwd_bwd`` on the configuration's operands (4 Mi elements, per-element bit-widths, RND, training):
    y bit-exact, dx / di / df within 1e-5 per element of the oracle's callable and its custom gradients
    (reference fixed_point_quantizer.py:142-150; KBI: f = b - i, :256-265), and bit-equal to the two separate
    launches.  i reaches below -f here, so SAT words with i + f < 0 are part of the case."""
    from hgq2_amd import _lib, ops

    n = 4 * 1024 * 1024
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(n, generator=g) * 2.0).requires_grad_(True)
    k = torch.randint(0, 2, (n,), generator=g).float() if overflow_mode != 'WRAP' else torch.ones(n)
    i = torch.randint(-2, 5, (n,), generator=g).float().requires_grad_(True)
    fb = torch.randint(0, 9, (n,), generator=g).float().requires_grad_(True)  # f, or b with kbi
    gy = torch.randn(n, generator=g)
    q = ofp.get_fixed_quantizer('RND', overflow_mode)
    want = q(x, k, i, fb - i if kbi else fb, True, None)
    want.backward(gy)
    mode = _lib.mode_bits('RND', overflow_mode, training=True, kbi=kbi)
    xd, kd, idv, fd, gd = (t.detach().to(dev) for t in (x, k, i, fb, gy))
    y, dx, di, dfb = ops.quantize_fwd_bwd(xd, kd, idv, fd, gd, mode, 1)
    assert torch.equal(y.cpu(), want.detach())
    for got, ref_g, name in ((dx, x.grad, 'dx'), (di, i.grad, 'di'), (dfb, fb.grad, 'df')):
        ref_g = torch.zeros(n) if ref_g is None else ref_g
        np.testing.assert_allclose(got.cpu().numpy(), ref_g.numpy(), rtol=RTOL, atol=1e-30, err_msg=f'{overflow_mode} kbi={kbi} {name}')
    y2, _, _ = ops.quantize_fwd(xd, kd, idv, fd, mode, 1, False)
    dx2, di2, dfb2 = ops.quantize_bwd(gd, xd, kd, idv, fd, mode, 1, True, True)
    for a, b in ((y, y2), (dx, dx2), (di, di2), (dfb, dfb2)):
        assert torch.equal(a, b)


@pytest.mark.parametrize('n,bw_shape,x_shape', [(4 * 1000 + 3, None, None), (7, None, None), (2, None, None),
                                               (None, (1, 24), (300, 24)), (None, (1, 1), (37, 5)), (None, (1, 6, 1), (9, 6, 10))])
@pytest.mark.parametrize('round_mode,overflow_mode', [('RND', 'WRAP'), ('TRN', 'SAT'), ('RND_CONV', 'SAT_SYM')])
def test_quantizer_fwd_bwd_in_one_launch_ragged_and_shared(dev, n, bw_shape, x_shape, round_mode, overflow_mode):
    """Sizes that are not a multiple of four, tiny inputs, a uint8 k, and bit-widths shared over axes (where the
    entry point runs the two passes): the same results as the separate forward and backward operators."""
    from hgq2_amd import _lib, ops

    g = torch.Generator().manual_seed(7)
    if x_shape is None:
        x_shape = bw_shape = (n,)
    x = (torch.randn(x_shape, generator=g) * 3).to(dev)
    gy = torch.randn(x_shape, generator=g).to(dev)
    k = torch.randint(0, 2, bw_shape, generator=g).to(torch.uint8).to(dev)
    i = torch.randint(-1, 4, bw_shape, generator=g).float().to(dev)
    f = torch.randint(0, 7, bw_shape, generator=g).float().to(dev)
    inner = 1
    for a in range(len(x_shape) - 1, -1, -1):
        if bw_shape[a] != 1:
            break
        inner *= x_shape[a]
    mode = _lib.mode_bits(round_mode, overflow_mode, training=True)
    y, dx, di, df = ops.quantize_fwd_bwd(x, k, i, f, gy, mode, inner)
    y2, _, _ = ops.quantize_fwd(x, k, i, f, mode, inner, False)
    dx2, di2, df2 = ops.quantize_bwd(gy, x, k, i, f, mode, inner, True, True)
    assert torch.equal(y, y2) and torch.equal(dx, dx2)
    if i.numel() == x.numel():
        assert torch.equal(di, di2) and torch.equal(df, df2)
    else:  # sums over the shared axes: the separate operator may add them in another (fixed) order
        scale = gy.abs().sum() * (math.log(2) * 8.0 + 1.0)
        assert float((di - di2).abs().max()) <= RTOL * float(scale) and float((df - df2).abs().max()) <= RTOL * float(scale)


@pytest.mark.parametrize('overflow_mode', ['SAT', 'SAT_SYM'])
@pytest.mark.parametrize('bw_shape', [(600, 24), (1, 24), (1, 1)])
def test_saturating_training_where_the_word_has_no_bits(dev, overflow_mode, bw_shape):
    """SAT / SAT_SYM in training with i + f < 0 on most entries (i in -6..0, f in 0..3): this build's definition of the
    case - the reference's bound formulas applied as they stand, upper bound first, every violated bound taking gradient
    (tests/test_oracle_pins.py::test_saturating_words_with_negative_total_width_are_defined_by_the_bounds) - values bit
    for bit and gradients to 1e-5 of the summed |terms|, with bit-widths per element, per column and shared."""
    from hgq2_amd import _lib, ops

    shape = (600, 24)
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(shape, generator=g) * 0.5)
    k = torch.randint(0, 2, bw_shape, generator=g).float()
    i = torch.randint(-6, 1, bw_shape, generator=g).float()
    f = torch.randint(0, 4, bw_shape, generator=g).float()
    if i.numel() == 1:
        i, f = torch.full(bw_shape, -2.0), torch.full(bw_shape, 1.0)
    assert float(((i + f) < 0).float().mean()) > 0.4
    gy = torch.randn(shape, generator=g)
    q = ofp.get_fixed_quantizer('RND', overflow_mode)
    xs = x.clone().requires_grad_(True)
    ie, fe = (t.expand(shape).clone().requires_grad_(True) for t in (i, f))   # per-element terms of the oracle
    want = q(xs, k.expand(shape), ie, fe, True, None)
    want.backward(gy)
    hom = tuple(a for a in range(2) if bw_shape[a] == 1)
    mode = _lib.mode_bits('RND', overflow_mode, training=True)
    xd = x.to(dev).requires_grad_(True)
    idv, fd = (t.reshape(-1).to(dev).requires_grad_(True) for t in (i, f))
    y, _, _ = ops.quantize(xd, k.reshape(-1).to(dev), idv, fd, mode, bw_inner=1)
    assert torch.equal(y.detach().cpu(), want.detach())
    y.backward(gy.to(dev))
    assert torch.equal(xd.grad.cpu(), xs.grad)
    for got, terms, name in ((idv.grad, ie.grad, 'di'), (fd.grad, fe.grad, 'df')):
        t64 = terms.double()
        want_g = t64.sum(dim=hom).reshape(-1) if hom else t64.reshape(-1)
        scale = t64.abs().sum(dim=hom).reshape(-1) if hom else t64.abs().reshape(-1)
        _close_scaled(got, want_g, scale, f'{overflow_mode} {bw_shape} {name}')


# --------------------------------------------------------------------------------------------------------------
# the stateless callable, driven as the reference drives it
# --------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize('x_shape,bw_shape', [((3000, 24), (1, 24)), ((700, 6, 10), (1, 6, 10)), ((513, 33), (1, 1)),
                                              ((64, 8, 16), (1, 8, 1)), ((40, 50), (40, 50))])
@pytest.mark.parametrize('overflow_mode', ['WRAP', 'SAT', 'SAT_SYM'])
def test_fixed_quantizer_callable_as_the_reference_calls_it(dev, x_shape, bw_shape, overflow_mode):
    """Reference src/hgq/quantizer/internal/fixed_point_quantizer.py:142-150: k, i, f are ``broadcast_to`` the
    input's shape, then ``q(x, k, i, f, training, None)``; :288,:405: ``q.round(x, f, False, None)``.  The callable of
    ``hgq2_amd.quantizer.fixed_point_ops`` must give the oracle's values bit for bit and its gradients to x and to the
    small bit-width tensors (autograd sums the broadcast back)."""
    from hgq2_amd.quantizer.fixed_point_ops import get_fixed_quantizer

    g = torch.Generator().manual_seed(sum(x_shape))
    x = torch.randn(x_shape, generator=g) * 3
    k = torch.randint(0, 2, bw_shape, generator=g).float()
    i = torch.randint(-1, 4, bw_shape, generator=g).float()
    f = torch.randint(0, 7, bw_shape, generator=g).float()
    gy = torch.randn(x_shape, generator=g)
    q_ref, q_dev = ofp.get_fixed_quantizer('RND', overflow_mode), get_fixed_quantizer('RND', overflow_mode)
    assert q_dev.round_mode == 'RND' and q_dev.stochastic is False

    def run(q, device, training, rounding_only):
        xs = x.clone().to(device).requires_grad_(True)
        ks = k.to(device)
        is_, fs = i.clone().to(device).requires_grad_(True), f.clone().to(device).requires_grad_(True)
        kb, ib, fb = (torch.broadcast_to(t, x_shape) for t in (ks, is_, fs))
        y = q.round(xs, fb, False, None) if rounding_only else q(xs, kb, ib, fb, training, None)
        if training:
            y.backward(gy.to(device))
        return y.detach().cpu(), xs.grad, is_.grad, fs.grad

    for training, rounding_only in ((True, False), (False, False), (True, True)):
        want = run(q_ref, 'cpu', training, rounding_only)
        got = run(q_dev, dev, training, rounding_only)
        want_y = want[0]
        if not training:
            kb, ib, fb = (torch.broadcast_to(t, x_shape) for t in (k, i, f))
            want_y = torch.where(kb + ib + fb > 0, want_y, torch.zeros_like(want_y))  # the reference applies this around the call
        assert torch.equal(got[0], want_y), f'values training={training} round={rounding_only}'
        if not training:
            continue
        np.testing.assert_allclose(got[1].cpu().numpy(), want[1].numpy(), rtol=RTOL, atol=1e-30)
        hom = tuple(a for a in range(len(x_shape)) if bw_shape[a] == 1 and x_shape[a] != 1)
        for gg, wg, name in ((got[2], want[2], 'di'), (got[3], want[3], 'df')):
            wg = torch.zeros(bw_shape) if wg is None else wg
            gg = torch.zeros(bw_shape) if gg is None else gg.cpu()
            # a sum over the broadcast axes: bound by the sum of |terms|, which is at most sum |gy| * max coefficient
            scale = gy.abs().sum(dim=hom, keepdim=True) * (math.log(2) * 2.0 ** i.clamp(min=0) + 1.0) if hom else wg.abs() + 1e-6
            _close_scaled(gg, wg, scale.expand(bw_shape) if hom else scale, f'{name} training={training} round={rounding_only}')


# --------------------------------------------------------------------------------------------------------------
# KBI WRAP with batch-shared bit-widths: training and calibration
# --------------------------------------------------------------------------------------------------------------
def _kbi_wrap_pair(dev, F, g):
    from hgq2_amd.config import QuantizerConfig
    from hgq2_amd.quantizer import Quantizer

    q = Quantizer(QuantizerConfig('kbi', 'datalane', overflow_mode='WRAP', round_mode='RND'))
    q(torch.zeros(4, F, device=dev), training=False)  # build on the device
    with torch.no_grad():
        q.quantizer._b.copy_(torch.randint(0, 9, (1, F), generator=g).float().to(dev))
        q.quantizer._i.copy_((torch.randint(-2, 3, (1, F), generator=g).float() + 0.3).to(dev))
    return q, twin.ref_quantizer(q)


def test_kbi_wrap_training_matches_oracle_with_many_row_chunks(dev):
    """Reference fixed_point_quantizer.py:277-288.  2000 rows of a [1, F] quantizer span several row chunks of the
    per-column kernels; integer bits exact over three steps, values exact, d/db within the sum bound."""
    g = torch.Generator().manual_seed(21)
    F = 16
    q, r = _kbi_wrap_pair(dev, F, g)
    assert tuple(q.quantizer._b.shape) == (1, F) and q.quantizer.overflow_mode == 'WRAP'
    x = torch.randn(2000, F, generator=g) * torch.logspace(-2, 2, F)
    x[:, 3] = 0.0
    x[:, 4:7] = x[:, 4:7].clamp(-0.25, 0.25)
    x[0, 4], x[1, 5], x[2, 6] = 1.0, -0.5, 4.0  # exact powers of two as column maxima (they stay so when halved)
    for step in range(3):
        xs = x * (0.5 ** step)
        xp, xr = xs.to(dev).requires_grad_(True), xs.clone().requires_grad_(True)
        gy = torch.randn(xs.shape, generator=g)
        yp, yr = q(xp, training=True), r(xr, training=True)
        assert torch.equal(q.quantizer._i.cpu(), r.quantizer._i.detach()), f'_i step {step}'
        assert torch.equal(yp.detach().cpu(), yr.detach()), f'values step {step}'
        q.quantizer._b.grad = r.quantizer._b.grad = None
        yp.backward(gy.to(dev))
        yr.backward(gy)
        np.testing.assert_allclose(xp.grad.cpu().numpy(), xr.grad.numpy(), rtol=RTOL, atol=1e-30)
        delta = (yr.detach() - xs).double()
        scale = (math.log(2) * delta.abs() * gy.double().abs()).sum(0, keepdim=True) + 1e-12
        _close_scaled(q.quantizer._b.grad, r.quantizer._b.grad, scale, f'd/db step {step}')
    assert torch.equal(q.quantizer._k.cpu(), r.quantizer._k)


def test_kbi_wrap_tracing_matches_oracle_with_many_row_chunks(dev):
    """Reference fixed_point_quantizer.py:289-300 through the calibration flag: integer bits only grow, rounding uses
    the new integer bits, the keep-negative flag collects negatives of the rounded values where b > 0."""
    from hgq2_amd.core import TrainingFlagWrapper

    g = torch.Generator().manual_seed(22)
    F = 16
    q, r = _kbi_wrap_pair(dev, F, g)
    with torch.no_grad():
        for inner in (q.quantizer, r.quantizer):
            inner._i.fill_(-1e9)
            inner._k.zero_()
    flag = TrainingFlagWrapper('tracing')
    base = torch.randn(1500, F, generator=g) * torch.logspace(-2, 1.5, F)
    base[:, 2] = base[:, 2].abs()            # a lane that never goes negative
    base[:, 7] = -base[:, 7].abs() * 1e-4    # negatives that round to zero for small f
    for scale in (0.25, 1.0, 0.5):
        xs = base * scale
        yp, yr = q(xs.to(dev), training=flag), r(xs, training=flag)
        assert torch.equal(yp.cpu(), yr), f'values at scale {scale}'
        assert torch.equal(q.quantizer._i.cpu(), r.quantizer._i.detach()), f'_i at scale {scale}'
        assert torch.equal(q.quantizer._k.cpu(), r.quantizer._k), f'_k at scale {scale}'
    assert int(r.quantizer._k.sum()) not in (0, F)  # both outcomes occur


# --------------------------------------------------------------------------------------------------------------
# the Quantizer wrapper with its optional stages
# --------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize('extras', [dict(scaler=4.0), dict(qnoise_factor=0.3), dict(affine=(0.5, -2.0)),
                                    dict(scaler=0.125, qnoise_factor=0.75, affine=(3.0, 1.0))])
@pytest.mark.parametrize('overflow_mode', ['WRAP', 'SAT'])
def test_quantizer_wrapper_scaler_qnoise_affine(dev, extras, overflow_mode):
    """Reference src/hgq/quantizer/quantizer.py:49-60 against the oracle twin: the inner quantizer's values are exact,
    the elementwise stages around it (one kernel pass in front, one behind, one IEEE operation per step of the reference)
    are fp32 ops in the same order, so the outputs are compared bit for bit in inference and in training."""
    from hgq2_amd.config import QuantizerConfig
    from hgq2_amd.quantizer import Quantizer

    g = torch.Generator().manual_seed(23)
    q = Quantizer(QuantizerConfig('kif', 'datalane', overflow_mode=overflow_mode, **extras))
    x = torch.randn(3000, 12, generator=g) * 3
    q(x.to(dev), training=False)
    with torch.no_grad():
        q.quantizer._f.copy_(torch.randint(1, 6, (1, 12), generator=g).float().to(dev))
        q.quantizer._i.copy_(torch.randint(0, 3, (1, 12), generator=g).float().to(dev))
    r = twin.ref_quantizer(q)
    with torch.no_grad():
        assert torch.equal(q(x.to(dev), training=False).cpu(), r(x, training=False))
    xp, xr = x.to(dev).requires_grad_(True), x.clone().requires_grad_(True)
    gy = torch.randn(x.shape, generator=g)
    yp, yr = q(xp, training=True), r(xr, training=True)
    assert torch.equal(yp.detach().cpu(), yr.detach())
    assert torch.equal(q.quantizer._i.cpu(), r.quantizer._i.detach())
    yp.backward(gy.to(dev))
    yr.backward(gy)
    np.testing.assert_allclose(xp.grad.cpu().numpy(), xr.grad.numpy(), rtol=RTOL, atol=1e-7)
    scale = gy.abs().sum(0, keepdim=True) * 64.0  # sum of |gy| x the largest coefficient any stage can contribute
    _close_scaled(q.quantizer._f.grad, r.quantizer._f.grad, scale, 'd/df')
    if overflow_mode == 'SAT':  # the integer bits are trainable unless the overflow mode is WRAP
        _close_scaled(q.quantizer._i.grad, r.quantizer._i.grad, scale, 'd/di')


@pytest.mark.parametrize('n,offset', [(4096, 0), (1001, 0), (1023, 1), (3, 0), (1, 2)])
@pytest.mark.parametrize('scaler,noise,affine', [(3.0, None, None), (None, 0.3, None), (None, None, (0.25, 0.5)), (0.7, 0.45, (3.0, -1.0))])
def test_quantizer_wrapper_kernels_equal_the_elementwise_operations(dev, n, offset, scaler, noise, affine):
    """``ops.quantizer_scale_div`` / ``ops.quantizer_tail`` against the same chain written as separate CPU tensor operations
    (reference src/hgq/quantizer/quantizer.py:49-60), values and gradients bit for bit, for sizes that are no multiple of
    four and arrays that are not 16-byte aligned."""
    from hgq2_amd import ops

    g = torch.Generator().manual_seed(n + offset)
    base = torch.randn(3, n + offset, generator=g) * 5
    x, xs, gy = (base[k, offset:].clone() for k in range(3))
    dev_of = lambda t: torch.zeros(t.numel() + offset, device=dev)[offset:].copy_(t)  # the same misalignment on the device
    if scaler is not None:
        xr = x.clone().requires_grad_(True)
        want = xr / scaler
        want.backward(gy)
        xd = dev_of(x).requires_grad_(True)
        got = ops.quantizer_scale_div(xd, scaler)
        got.backward(dev_of(gy))
        assert torch.equal(got.detach().cpu(), want.detach()) and torch.equal(xd.grad.cpu(), xr.grad)
    qr, xsr = x.clone().requires_grad_(True), xs.clone().requires_grad_(True)
    out = qr
    if scaler is not None:
        out = out * scaler
    if noise is not None:
        out = xsr + noise * (out - xsr)
    if affine is not None:
        out = out * affine[0] + affine[1]
    out.backward(gy)
    qd, xsd = dev_of(x).requires_grad_(True), dev_of(xs).requires_grad_(True)
    got = ops.quantizer_tail(qd, xsd, scaler, noise, affine)
    got.backward(dev_of(gy))
    assert torch.equal(got.detach().cpu(), out.detach())
    assert torch.equal(qd.grad.cpu(), qr.grad)
    if noise is not None:
        assert torch.equal(xsd.grad.cpu(), xsr.grad)
    else:
        assert xsd.grad is None


# --------------------------------------------------------------------------------------------------------------
# configurations 3 and 4: backward at full size
# --------------------------------------------------------------------------------------------------------------
def _abs_sum_scales(contract, x_q, w_q, dz):
    """Sum of |terms| of the three gradients of a bilinear contraction y = contract(x, w): autograd of the same
    contraction on absolute operands, in float64."""
    xa = x_q.detach().double().abs().requires_grad_(True)
    wa = w_q.detach().double().abs().requires_grad_(True)
    contract(xa, wa).backward(dz.detach().double().abs())
    return xa.grad, wa.grad


def _layer_backward_check(dev, layer, r, x, g, contract, what, second_path=False):
    """One training forward + backward of a product layer and its oracle twin from the same input and upstream
    gradient; every gradient compared."""
    from hgq2_amd.train import model_loss

    xp, xr = x.to(dev).requires_grad_(True), x.clone().requires_grad_(True)
    yp = layer(xp, training=True)
    yr = r(xr, training=True)
    gy = torch.randn(yr.shape, generator=g)
    model_loss(layer, (yp * gy.to(dev)).sum()).backward()
    ((yr * gy.double()).sum() + r.extra_loss()).backward()
    assert torch.equal(layer.iq.quantizer._i.cpu(), r.iq.quantizer._i.detach()), f'{what}: tracked integer bits'
    assert int(layer.ebops.cpu().view(torch.int32)) == int(r.ebops_value), f'{what}: EBOPs'
    # forward: each output is a sum over the contraction
    with torch.no_grad():  # the operands of the contraction, for the sum-of-|terms| scales
        xq = ofp.fixed_round(x, torch.broadcast_to(r.iq.quantizer.f.detach(), x.shape), r.iq.quantizer.round_mode, False)
        wq = r.kq.last
        y_scale = contract(xq.double().abs(), wq.double().abs()) + 1e-6
    _close_scaled(yp, yr, y_scale, f'{what}: output')
    dz = gy.double() * (yr.detach() > 0) if r.activation == 'relu' else gy.double()
    sx, sw = _abs_sum_scales(contract, xq, wq, dz)
    if second_path:
        # batch-norm folding: x also reaches the loss through the batch statistics, a path the sum above does not see
        # (it alone carries the gradient of a row whose outputs are all inactive); its terms are bounded through the result
        sx = sx + xr.grad.detach().double().abs() + xr.grad.detach().double().abs().mean()
    _close_scaled(xp.grad, xr.grad, sx + 1e-9, f'{what}: dx')
    return dz, sw, yr.detach().float()


class _TapQuantizer(ref.RefQuantizer):
    """Keeps the last result (the quantized kernel that entered the contraction)."""

    def __call__(self, x, training=None):
        out = super().__call__(x, training=training)
        self.last = out.detach()
        return out


@pytest.mark.parametrize('kind', ['particle', 'conv'])
def test_full_size_backward_matches_oracle(dev, acc64, kind):
    """The per-particle network (4096 x 64 x 16 -> 64 -> 32 -> mean -> 5) and the image network (1024 x 28 x 28 x 1,
    two 3x3x32 convolutions, 10 outputs) at full size, layer by layer from the oracle's activations: output, dx and
    the gradients of kernel, bias, batch-norm scale and every bit-width variable."""
    import torch.nn.functional as F

    from hgq2_amd.utils import models

    g = torch.Generator().manual_seed(51)
    torch.manual_seed(51)
    if kind == 'particle':
        x = torch.randn(4096, 64, 16, generator=g)
        model = models.particle_mlp(device=dev)
    else:
        x = torch.rand(1024, 28, 28, 1, generator=g)
        model = models.conv_stack(device=dev)
    with torch.no_grad():
        model(x.to(dev), training=True)  # build, adapt the tracked bits
    from tests.test_gpu_more_layers import _perturb

    _perturb(model, g)
    h = x
    for layer in model.layers:
        if isinstance(layer, models.PARAMETER_FREE):
            h = layer.host_fn(h)
            continue
        name = layer.__class__.__name__
        for p in layer.parameters():
            p.grad = None
        if name == 'QConv2D':
            r = twin.ref_conv2d(layer)
            contract = lambda a, w: F.conv2d(a.permute(0, 3, 1, 2), w.permute(3, 2, 0, 1)).permute(0, 2, 3, 1)  # noqa: E731
        elif name == 'QEinsumDenseBatchnorm':
            r = twin.ref_einsum_dense_bn(layer, tuple(h.shape))
            contract = lambda a, w: torch.einsum('bpf,fh->bph', a, w)  # noqa: E731
        else:
            r = twin.ref_dense(layer)
            contract = lambda a, w: a @ w  # noqa: E731
        r.kq.__class__ = _TapQuantizer
        what = f'{kind}/{layer.name}'
        dz, sw, h_next = _layer_backward_check(dev, layer, r, h, g, contract, what, second_path=name == 'QEinsumDenseBatchnorm')
        # kernel: the straight-through gradient of the quantized kernel is the contraction's weight gradient
        named = [('kernel', layer._kernel, r.kernel), ('bias', layer.bias, r.bias), ('iq._f', layer.iq.quantizer._f, r.iq.quantizer._f),
                 ('kq._b', layer.kq.quantizer._b, r.kq.quantizer._b), ('kq._i', layer.kq.quantizer._i, r.kq.quantizer._i),
                 ('bq._b', layer.bq.quantizer._b, r.bq.quantizer._b), ('bq._i', layer.bq.quantizer._i, r.bq.quantizer._i)]
        if name == 'QEinsumDenseBatchnorm':
            named.append(('gamma', layer.bn_gamma, r.gamma))
        for vname, p, rv in named:
            if rv.grad is None:
                assert p.grad is None or float(p.grad.abs().max()) == 0.0, f'{what}: {vname} should have no gradient'
                continue
            assert p.grad is not None, f'{what}: {vname} has no gradient'
            if vname == 'kernel' and name != 'QEinsumDenseBatchnorm':
                _close_scaled(p.grad, rv.grad, sw + 1e-9, f'{what}: d{vname}')
            elif vname == 'bias' and name != 'QEinsumDenseBatchnorm':
                red = tuple(range(dz.dim() - 1))
                _close_scaled(p.grad, rv.grad, dz.abs().sum(dim=red) + 1e-9, f'{what}: d{vname}')
            else:
                _close_tensor(p.grad, rv.grad, f'{what}: d{vname}')
        h = h_next  # continue from the oracle's activations


# ---- stochastic rounding (round modes S_RND / S_RND_CONV)
@pytest.mark.parametrize('overflow_mode', ['WRAP', 'SAT', 'SAT_SYM'])
@pytest.mark.parametrize('bw_shape', [None, (1, 37), ()])
def test_stochastic_rounding_kernels_match_oracle(dev, overflow_mode, bw_shape):
    """The training-mode forward and surrogate backward with the draw named by (seed, offset): values bit-exact against
    the oracle's restatement of the same generator, gradients to 1e-5, for per-element, per-column and scalar bit-widths."""
    from hgq2_amd import _lib, ops

    g = torch.Generator().manual_seed(77)
    x = torch.randn(301, 37, generator=g) * 3
    shape = tuple(x.shape) if bw_shape is None else bw_shape
    k = torch.randint(0, 2, shape, generator=g).float()
    i = torch.randint(-1, 3, shape, generator=g).float()
    f = torch.randint(0, 6, shape, generator=g).float()
    seed, offset = 2**40 + 12345, 2**33 + 9
    q = ofp.get_fixed_quantizer("S_RND", overflow_mode)
    xr, ir, fr = x.clone().requires_grad_(True), i.clone().requires_grad_(True), f.clone().requires_grad_(True)
    want = q(xr, k.expand(x.shape), ir.expand(x.shape), fr.expand(x.shape), True, (seed, offset))
    up = torch.randn(x.shape, generator=g)
    (want * up).sum().backward()
    from hgq2_amd.quantizer.internal.base import bw_layout

    inner = bw_layout(shape, tuple(x.shape))[1]
    xd = x.to(dev).requires_grad_(True)
    idv, fd = i.reshape(-1).to(dev).requires_grad_(True), f.reshape(-1).to(dev).requires_grad_(True)
    mode = _lib.mode_bits('S_RND', overflow_mode, training=True)
    got, _, _ = ops.quantize_stochastic(xd, k.reshape(-1).to(dev), idv, fd, mode, seed, offset, bw_inner=inner)
    assert torch.equal(got.detach().cpu(), want.detach()), float((got.detach().cpu() - want.detach()).abs().max())
    (got * up.to(dev)).sum().backward()
    assert torch.equal(xd.grad.cpu(), xr.grad)
    for name, a, b in (('di', idv.grad, ir.grad), ('df', fd.grad, fr.grad)):
        if b is None:  # WRAP in training is rounding only: nothing reaches the integer bits
            assert a is None or float(a.abs().max()) == 0.0, name
            continue
        b = b.reshape(-1)
        scale = float(b.abs().max()) + 1e-30
        terms = math.log(2.0) * float(up.abs().sum()) / max(b.numel(), 1) if bw_shape is not None else 0.0  # sum of |terms| per entry, about
        assert float((a.cpu() - b).abs().max()) <= 1e-5 * (scale + terms), name
    # another offset is another draw; the same pair repeats it
    again, _, _ = ops.quantize_stochastic(xd.detach(), k.reshape(-1).to(dev), idv.detach(), fd.detach(), mode, seed, offset, bw_inner=inner)
    other, _, _ = ops.quantize_stochastic(xd.detach(), k.reshape(-1).to(dev), idv.detach(), fd.detach(), mode, seed, offset + 1, bw_inner=inner)
    assert torch.equal(again, got.detach()) and not torch.equal(other, got.detach())


@pytest.mark.parametrize('q_type,overflow_mode,round_mode', [('kif', 'WRAP', 'S_RND'), ('kif', 'SAT', 'S_RND_CONV'), ('kbi', 'WRAP', 'S_RND'),
                                                             ('kbi', 'SAT_SYM', 'S_RND')])
def test_stochastic_quantizer_classes_follow_the_oracle(dev, q_type, overflow_mode, round_mode):
    """KIF / KBI quantizer layers with a stochastic round mode: two training calls (the generator advances), the tracked
    integer bits, the gradients, a tracing call and inference (both deterministic) against the oracle twin."""
    from hgq2_amd.quantizer import Quantizer, QuantizerConfig

    g = torch.Generator().manual_seed(78)
    x = torch.randn(700, 24, generator=g) * 2
    conf = QuantizerConfig(q_type, 'datalane', overflow_mode=overflow_mode, round_mode=round_mode)
    q = Quantizer(conf)
    q.quantizer._seed = 4242  # (drawn at random at construction, like the reference's; fixed here before the build uses it)
    q(x.to(dev), training=True)  # build
    r = twin.ref_quantizer(q)
    assert q.quantizer.stochastic and r.quantizer.seed_gen is not None
    for step in range(2):
        xp, xr = x.to(dev).requires_grad_(True), x.clone().requires_grad_(True)
        yp, yr = q(xp, training=True), r(xr, training=True)
        assert torch.equal(yp.detach().cpu(), yr.detach()), f'step {step}'
        assert torch.equal(q.quantizer._i.detach().cpu(), r.quantizer._i.detach()), f'step {step}'
        up = torch.randn(x.shape, generator=g)
        for v in (q.quantizer._i, q.quantizer._third(), r.quantizer._i, r.quantizer._f if q_type == 'kif' else r.quantizer._b):
            v.grad = None
        (yp * up.to(dev)).sum().backward()
        (yr * up).sum().backward()
        assert torch.equal(xp.grad.cpu(), xr.grad)
        want = (r.quantizer._f if q_type == 'kif' else r.quantizer._b).grad
        got = q.quantizer._third().grad
        bound = 1e-5 * (float(want.abs().max()) + math.log(2.0) * float(up.abs().sum()) / want.numel())
        assert float((got.cpu() - want).abs().max()) <= bound, f'step {step}'
    assert q.quantizer._seed_gen.offset == r.quantizer.seed_gen.offset == 3
    from hgq2_amd.core import TrainingFlagWrapper

    with torch.no_grad():
        assert torch.equal(q(x.to(dev), training=TrainingFlagWrapper('tracing')).cpu(), r(x, training=TrainingFlagWrapper('tracing')))
        assert torch.equal(q(x.to(dev), training=False).cpu(), r(x, training=False))
    assert q.quantizer._seed_gen.offset == 3  # no draw outside training


def test_scaler_division_is_correctly_rounded(dev):
    """``inputs / scaler`` (reference src/hgq/quantizer/quantizer.py:50-51) with a scaler that is no power of two: the quotient
    has to be the correctly rounded one - a multiplication by 1 / scaler is an ulp off for about one value in eight, which
    stochastic rounding turns into a different quantized value for some of them."""
    from hgq2_amd.quantizer import Quantizer, QuantizerConfig

    g = torch.Generator().manual_seed(31)
    x = torch.randn(20000, 24, generator=g) * 30
    q = Quantizer(QuantizerConfig('kif', 'datalane', overflow_mode='SAT', round_mode='S_RND', scaler=3.0))
    q.quantizer._seed = 99
    q(x.to(dev), training=True)
    r = twin.ref_quantizer(q)
    want_in = x / 3.0
    assert not torch.equal(want_in, x * torch.tensor(1.0 / 3.0)), 'the data must tell the two apart'
    for step in range(2):
        yp, yr = q(x.to(dev), training=True), r(x, training=True)
        assert torch.equal(yp.cpu(), yr), f'step {step}: {int((yp.cpu() != yr).sum())} values differ'


def test_host_side_draws_refuse_graph_capture(dev):
    """A draw whose offset travels as a launch argument would repeat on every replay: `next()` without a device refuses a
    capturing stream, and so does the first device draw of a generator (its counter would be created by a recorded launch)."""
    from hgq2_amd.quantizer.fixed_point_ops import SeedGenerator

    for args in ((), (dev,)):
        gen = SeedGenerator(1)
        graph = torch.cuda.CUDAGraph()
        x = torch.zeros(8, device=dev)
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            with pytest.raises(RuntimeError, match='capture'):
                with torch.cuda.graph(graph, stream=s):
                    x.add_(1.0)
                    gen.next(*args)
        torch.cuda.current_stream().wait_stream(s)


def test_device_side_draw_counter_gives_the_host_counters_offsets(dev):
    """The draws of a seed generator on the GPU - offset = device counter + draws since it was advanced - are those of the
    host counter 1, 2, 3, ...: values equal the kernel called with the explicit pair, before and after advances."""
    from hgq2_amd import _lib, ops
    from hgq2_amd.quantizer.fixed_point_ops import SeedGenerator

    g = torch.Generator().manual_seed(11)
    x = (torch.randn(4096, generator=g) * 3).to(dev)
    k, i, f = torch.ones(1, device=dev), torch.full((1,), 3.0, device=dev), torch.full((1,), 2.0, device=dev)
    mode = _lib.mode_bits('RND', 'SAT', training=True)
    gen = SeedGenerator(77)
    for step in range(1, 7):
        if step in (3, 4, 6):
            ops.advance_seed_generators()
        seed, n, base = gen.next(dev)
        got, _, _ = ops.quantize_stochastic(x, k, i, f, mode, seed, n, bw_inner=x.numel(), base=base)
        want, _, _ = ops.quantize_stochastic(x, k, i, f, mode, 77, step, bw_inner=x.numel())
        assert torch.equal(got, want), step
        assert gen.offset == step and int(base) + gen._drawn == step
    # the backward pass repeats the draw the forward pass made, also when the counter has moved on in between
    xr = x.clone().requires_grad_(True)
    seed, n, base = gen.next(dev)
    y, _, _ = ops.quantize_stochastic(xr, k, i, f, mode, seed, n, bw_inner=x.numel(), base=base)
    ops.advance_seed_generators()
    gen.next(dev)
    y.sum().backward()
    xe = x.clone().requires_grad_(True)
    ye, _, _ = ops.quantize_stochastic(xe, k, i, f, mode, 77, 7, bw_inner=x.numel())
    ye.sum().backward()
    assert torch.equal(y, ye) and torch.equal(xr.grad, xe.grad)


def test_stochastic_rounding_in_a_replayed_graph_draws_anew(dev):
    """A training step with S_RND data quantizers recorded into a HIP graph: every replay draws as the same step run
    eagerly would - the losses of N replays are those of the same N eager steps of a twin model - and two replays on the
    same batch do not repeat each other's draw."""
    import numpy as np

    from hgq2_amd import ops
    from hgq2_amd.core import Sequential, set_default_device
    from hgq2_amd.layers import QDense
    from hgq2_amd.quantizer.config import QuantizerConfigScope
    from hgq2_amd.train import SGD, GraphedTrainStep, model_loss

    set_default_device(dev)

    def build():
        np.random.seed(31)  # the quantizers take their seeds from numpy's generator (reference: internal/base.py seed default)
        torch.manual_seed(2)
        with QuantizerConfigScope(place='datalane', round_mode='S_RND'):
            model = Sequential([QDense(24, activation='relu'), QDense(6)])
        model(x, training=False)
        return model

    g = torch.Generator().manual_seed(4)
    x = torch.randn(256, 12, generator=g).to(dev)
    y = torch.randint(0, 6, (256,), generator=g).to(dev)
    a, b = build(), build()
    for pa, pb in zip(a.parameters(), b.parameters()):
        assert torch.equal(pa, pb)
    gens = [m.seed_gen for m in a.modules() if getattr(m, 'seed_gen', None) is not None]
    assert gens, 'no stochastic quantizer in the model'
    opt_a, opt_b = SGD(a.parameters(), lr=0.05), SGD(b.parameters(), lr=0.05)
    warmup, replays = 2, 4
    step_a = GraphedTrainStep(a, ops.sparse_ce, opt_a, x, y, warmup=warmup)
    losses = [step_a().item() for _ in range(replays)]
    want = []
    for _ in range(warmup + replays):  # the recording itself runs nothing
        opt_b.zero_grad()
        with ops.overlap_ebops():
            loss = model_loss(b, ops.sparse_ce(b(x, training=True), y))
            opt_b.backward(loss)
            opt_b.step()
        want.append(loss.item())
    torch.cuda.synchronize()
    # (the shared bit-widths' gradients of the stochastic kernels are added with float atomics: the trajectories agree to
    # rounding, not to the bit; a replay that repeated a draw would be off by the rounding noise itself, ~1e-3)
    assert all(abs(a - b) <= 1e-5 * abs(b) for a, b in zip(losses, want[warmup:])), (losses, want)
    assert len(set(losses)) > 1
