"""GPU parity of the HIP kernels (through torch.library -> ctypes -> C ABI) against the CPU oracle.

Bar: quantized values, tracked integer bits and EBOPs bit-exact; contractions and gradients
within 1e-5 relative (fp32; the reference statement is evaluated in float64 where a sum is
involved so that the tolerance measures the kernel, not the checker)."""

import numpy as np
import pytest
import torch

from oracle import fixed_point as ofp
from oracle import hgq_ref as ref

pytestmark = pytest.mark.gpu

ROUND = ('TRN', 'RND', 'RND_CONV')
OVER = ('WRAP', 'SAT', 'SAT_SYM')
RTOL = 1e-5


def _ops():
    from hgq2_amd import _lib, ops

    return _lib, ops


def _rand_kif(shape, g, kbi=False):
    k = torch.randint(0, 2, shape, generator=g).float()
    i = torch.randint(-2, 5, shape, generator=g).float()
    f = torch.randint(0, 9, shape, generator=g).float()
    if kbi:
        return k, i, i + f  # b = i + f >= 0
    return k, i, f


def _assert_close_sum(got, want64, scale64, what):
    """|got - want| <= RTOL * sum|terms| : a relative bound that is meaningful under cancellation."""
    err = (got.double().cpu() - want64).abs()
    tol = RTOL * scale64 + 1e-30
    assert torch.all(err <= tol), f'{what}: max err {err.max().item():.3e} tol {tol.min().item():.3e}'


@pytest.mark.parametrize('round_mode', ROUND)
@pytest.mark.parametrize('overflow_mode', OVER)
@pytest.mark.parametrize('training', (False, True))
@pytest.mark.parametrize('n', (1, 3, 4099, 1 << 16))
def test_quantize_per_element_values(dev, round_mode, overflow_mode, training, n):
    _lib, ops = _ops()
    g = torch.Generator().manual_seed(n)
    x = torch.randn(n, generator=g) * 4
    x[::7] = torch.round(x[::7] * 8) / 8 + 1 / 16  # exact ties for small f
    k, i, f = _rand_kif((n,), g)
    want = ofp.get_fixed_quantizer(round_mode, overflow_mode)(x, k, i, f, training, None)
    if not training:
        want = torch.where(k + i + f > 0, want, torch.zeros_like(want))
    mode = _lib.mode_bits(round_mode, overflow_mode, training=training)
    y, _, _ = ops.quantize(x.to(dev), k.to(dev), i.to(dev), f.to(dev), mode)
    assert torch.equal(y.cpu(), want)
    # uint8 k and raw (un-rounded) variables
    noise = (torch.rand(n, generator=g) - 0.5) * 0.8
    y2, _, _ = ops.quantize(x.to(dev), k.to(torch.uint8).to(dev), (i + noise).to(dev), (f - noise).to(dev),
                            mode | _lib.MODE_ROUND_PARAMS)
    assert torch.equal(y2.cpu(), want)


@pytest.mark.parametrize('overflow_mode', OVER)
@pytest.mark.parametrize('kbi', (False, True))
def test_quantize_per_element_gradients(dev, overflow_mode, kbi):
    _lib, ops = _ops()
    n = 50000
    g = torch.Generator().manual_seed(7)
    x = (torch.randn(n, generator=g) * 4).requires_grad_(True)
    k, i, fb = _rand_kif((n,), g, kbi)
    i.requires_grad_(True), fb.requires_grad_(True)
    f = fb - i if kbi else fb
    y = ofp.get_fixed_quantizer('RND', overflow_mode)(x, k, i, f, True, None)
    gy = torch.randn(n, generator=g)
    y.backward(gy)
    mode = _lib.mode_bits('RND', overflow_mode, training=True, kbi=kbi)
    xd = x.detach().to(dev).requires_grad_(True)
    idv = i.detach().to(dev).requires_grad_(True)
    fd = fb.detach().to(dev).requires_grad_(True)
    yd, _, _ = ops.quantize(xd, k.to(dev), idv, fd, mode)
    assert torch.equal(yd.detach().cpu(), y.detach())
    yd.backward(gy.to(dev))
    for got, want, name in ((xd.grad, x.grad, 'dx'), (idv.grad, i.grad, 'di'), (fd.grad, fb.grad, 'dfb')):
        want = torch.zeros(n) if want is None else want
        np.testing.assert_allclose(got.cpu().numpy(), want.numpy(), rtol=RTOL, atol=1e-30, err_msg=name)


@pytest.mark.parametrize('shape,bw_shape', [((4096, 16), (1, 16)), ((1000, 7), (1, 7)), ((64, 12, 20), (1, 12, 20)),
                                            ((3000,), ()), ((33, 5, 8), (1, 1, 1)), ((50, 6, 4), (1, 6, 1))])
@pytest.mark.parametrize('overflow_mode', ('WRAP', 'SAT'))
def test_quantize_broadcast_bitwidths(dev, shape, bw_shape, overflow_mode):
    """Bit-widths shared along the homogeneous axes: values, abs-max / any-negative trackers, reduced gradients."""
    _lib, ops = _ops()
    g = torch.Generator().manual_seed(11)
    x = (torch.randn(shape, generator=g) * 3).requires_grad_(True)
    k, i, f = _rand_kif(bw_shape, g)
    i.requires_grad_(True), f.requires_grad_(True)
    q = ofp.get_fixed_quantizer('RND', overflow_mode)
    kb, ib, fb = (torch.broadcast_to(t, shape) for t in (k, i, f))
    y = q(x, kb, ib, fb, True, None)
    gy = torch.randn(shape, generator=g)
    y.backward(gy)
    bw_size = max(1, int(np.prod(bw_shape)))
    # position of the heterogeneous block -> (bw_size, bw_inner)
    inner = 1
    for ax in range(len(shape) - 1, -1, -1):
        if len(bw_shape) and bw_shape[ax] != 1:
            break
        inner *= shape[ax]
    if bw_size == 1:
        inner = 1
    mode = _lib.mode_bits('RND', overflow_mode, training=True)
    xd = x.detach().to(dev).requires_grad_(True)
    idv = i.detach().reshape(-1).to(dev).requires_grad_(True)
    fd = f.detach().reshape(-1).to(dev).requires_grad_(True)
    yd, amax, neg = ops.quantize(xd, k.reshape(-1).to(dev), idv, fd, mode, bw_inner=inner, track=True)
    assert torch.equal(yd.detach().cpu(), y.detach())
    hom = tuple(a for a in range(len(shape)) if not len(bw_shape) or bw_shape[a] == 1)
    want_amax = torch.amax(y.detach().abs(), dim=hom).reshape(-1)
    want_neg = torch.amax((y.detach() < 0).int(), dim=hom).reshape(-1)
    # the trackers come as one entry per bit-width entry, or as slices [n_slices, bw_size] that the
    # integer-bit update combines (non-negative floats order like their bit patterns)
    amax, neg = amax.view(-1, bw_size).amax(0), neg.view(-1, bw_size).amax(0)
    assert torch.equal(amax.view(torch.float32).cpu(), want_amax)
    assert torch.equal(neg.cpu(), want_neg.int())
    yd.backward(gy.to(dev))
    np.testing.assert_allclose(xd.grad.cpu().numpy(), x.grad.numpy(), rtol=RTOL, atol=1e-30)
    # reduced gradients: float64 statement of the same per-element terms
    x64, gy64 = x.detach().double(), gy.double()
    delta = y.detach().double() - x64
    over = (y.detach() != ofp.fixed_round(x.detach(), fb, 'RND', False))
    f_terms = torch.where(over, torch.zeros_like(delta), -np.log(2) * delta * gy64)
    if overflow_mode == 'WRAP':
        want_df = f_terms.sum(dim=hom).reshape(-1)
        scale = f_terms.abs().sum(dim=hom).reshape(-1)
        _assert_close_sum(fd.grad, want_df, scale, 'df')
        assert torch.all(idv.grad == 0)
    else:
        # the oracle's own per-element terms (bit-widths expanded to leaves of the input's shape), summed in float64
        ie, fe = (t.detach().expand(shape).clone().requires_grad_(True) for t in (ib, fb))
        q(x.detach(), kb, ie, fe, True, None).backward(gy)
        for got, terms, name in ((fd.grad, fe.grad, 'df'), (idv.grad, ie.grad, 'di')):
            t64 = terms.double()
            _assert_close_sum(got, t64.sum(dim=hom).reshape(-1), t64.abs().sum(dim=hom).reshape(-1), name)


def test_wrap_track_i_matches_reference_recurrence(dev):
    _lib, ops = _ops()
    g = torch.Generator().manual_seed(3)
    q = ref.default_quantizer('datalane', (None, 40), q_type='kif', overflow_mode='WRAP')
    with torch.no_grad():
        q.quantizer._f.copy_(torch.randint(0, 9, (1, 40), generator=g).float())
        q.quantizer._i.copy_(torch.randint(-3, 3, (1, 40), generator=g).float() + 0.37)
    x = torch.randn(512, 40, generator=g) * torch.logspace(-2, 2, 40)
    x[:, 5] = 0.0
    x[:, 6] = 2.0 - 2.0 ** -float(q.quantizer._f[0, 6])  # exactly at 2**1 - 2**-f
    i_dev = q.quantizer._i.detach().clone().reshape(-1).to(dev)
    f_dev = q.quantizer._f.detach().clone().reshape(-1).to(dev)
    k_dev = q.quantizer._k.reshape(-1).to(dev)
    mode = _lib.mode_bits('RND', 'WRAP', training=True, round_params=True)
    for _ in range(3):
        want_y = q(x, training=True)
        y, amax, _ = ops.quantize(x.to(dev), k_dev, i_dev, f_dev, mode, track=True)
        ops.wrap_track_i_(amax, i_dev, f_dev, 0.01, mode)
        assert torch.equal(y.cpu(), want_y.detach())
        assert torch.equal(i_dev.cpu(), q.quantizer._i.detach().reshape(-1))
        x = x * 0.5


@pytest.mark.parametrize('rows,K,N,P', [(16384, 16, 64, 1), (1000, 64, 32, 1), (777, 32, 5, 1), (512, 12, 8, 1),
                                        (64 * 30, 16, 64, 64), (12 * 50, 8, 8, 12), (300, 7, 3, 1), (256, 40, 33, 1)])
@pytest.mark.parametrize('act', ('relu', None))
def test_qdense_forward_backward(dev, rows, K, N, P, act):
    _lib, ops = _ops()
    g = torch.Generator().manual_seed(rows + K)
    x = (torch.randn(rows, K, generator=g) * 2).requires_grad_(True)
    f = torch.randint(0, 7, (P, K), generator=g).float().requires_grad_(True)
    qw = (torch.round(torch.randn(K, N, generator=g) * 16) / 32).requires_grad_(True)
    qb = (torch.round(torch.randn(N, generator=g) * 16) / 32).requires_grad_(True)
    fb = f.repeat(rows // P, 1)
    rx = ofp.get_fixed_quantizer('RND', 'WRAP').round(x, fb, False, None)
    z = rx.double() @ qw.double() + qb.double()
    y = torch.relu(z) if act else z
    gy = torch.randn(rows, N, generator=g)
    y.backward(gy.double())
    mode = _lib.mode_bits('RND', 'WRAP', training=True)
    xd = x.detach().to(dev).requires_grad_(True)
    fd = f.detach().to(dev).requires_grad_(True)
    wd = qw.detach().to(dev).requires_grad_(True)
    bd = qb.detach().to(dev).requires_grad_(True)
    kd = torch.ones(P, K, device=dev)
    idv = torch.zeros(P, K, device=dev)
    yd, amax = ops.qdense(xd, kd, idv, fd, wd, bd, _lib.ACT_RELU if act else _lib.ACT_NONE, mode, P, True)
    scale = (rx.detach().double().abs() @ qw.detach().double().abs()) + qb.detach().double().abs()
    _assert_close_sum(yd.detach(), y.detach(), scale, 'y')
    want_amax = rx.detach().abs().reshape(rows // P, P, K).amax(dim=0).reshape(-1)
    assert torch.equal(amax.view(torch.float32).reshape(-1, P * K).amax(0).cpu(), want_amax)
    # The kernel's relu mask comes from its own fp32 output; rows where the sign of the
    # pre-activation is not decided at fp32 accuracy are excluded from the gradient check.
    yd.backward(gy.to(dev))
    if act:
        decided = (z.detach().abs() > RTOL * scale).all(dim=1)
    else:
        decided = torch.ones(rows, dtype=torch.bool)
    dz = gy.double() * ((z.detach() > 0) if act else 1.0)
    dx_scale = dz.abs() @ qw.detach().double().abs().T
    err = (xd.grad.cpu().double() - x.grad.double()).abs()
    assert torch.all(err[decided] <= RTOL * dx_scale[decided] + 1e-30)
    if bool(decided.all()):
        _assert_close_sum(wd.grad, qw.grad.double(), rx.detach().double().abs().T @ dz.abs(), 'dqw')
        _assert_close_sum(bd.grad, qb.grad.double(), dz.abs().sum(0), 'dqb')
        delta = rx.detach().double() - x.detach().double()
        terms = (-np.log(2) * delta * x.grad.double()).reshape(rows // P, P, K)
        _assert_close_sum(fd.grad.reshape(-1), terms.sum(0).reshape(-1), terms.abs().sum(0).reshape(-1) + 1e-12, 'df')


def test_qdense_exact_in_small_bitwidth_regime(dev):
    """Operands with few significant bits: every product and partial sum is exact in fp32, so the
    contraction must be bit-identical whatever the accumulation order."""
    _lib, ops = _ops()
    g = torch.Generator().manual_seed(5)
    x = torch.randn(4096, 64, generator=g) * 2
    f = torch.full((1, 64), 3.0)
    qw = torch.round(torch.randn(64, 64, generator=g) * 8) / 16
    qb = torch.round(torch.randn(64, generator=g) * 8) / 16
    want = torch.relu(ofp.fixed_round(x, f.expand_as(x), 'RND', False) @ qw + qb)
    mode = _lib.mode_bits('RND', 'WRAP', training=True)
    y, _ = ops.qdense(x.to(dev), torch.ones(1, 64, device=dev), torch.zeros(1, 64, device=dev), f.to(dev), qw.to(dev),
                      qb.to(dev), _lib.ACT_RELU, mode, 1, False)
    assert torch.equal(y.cpu(), want)


def test_qdense_large_shapes_forward_only(dev):
    _lib, ops = _ops()
    g = torch.Generator().manual_seed(9)
    x = torch.randn(500, 300, generator=g)
    f = torch.randint(2, 6, (1, 300), generator=g).float()
    qw = torch.round(torch.randn(300, 130, generator=g) * 16) / 32
    want = ofp.fixed_round(x, f.expand_as(x), 'RND', False).double() @ qw.double()
    mode = _lib.mode_bits('RND', 'WRAP', training=True)
    y, _ = ops.qdense(x.to(dev), torch.ones(1, 300, device=dev), torch.zeros(1, 300, device=dev), f.to(dev), qw.to(dev),
                      None, _lib.ACT_NONE, mode, 1, False)
    scale = x.double().abs() @ qw.double().abs()
    _assert_close_sum(y, want, scale, 'y')


def test_dense_ebops_exact_and_gradients(dev):
    _lib, ops = _ops()
    g = torch.Generator().manual_seed(13)
    layer = ref.RefMLP(dims=(24, 10)).layers[0]
    with torch.no_grad():
        layer.iq.quantizer._f.copy_(torch.randint(-3, 7, (1, 24), generator=g).float() + 0.2)
        layer.iq.quantizer._i.copy_(torch.randint(-2, 4, (1, 24), generator=g).float() - 0.3)
        layer.kq.quantizer._b.copy_(torch.randint(0, 9, (24, 10), generator=g).float() + 0.1)
        layer.bq.quantizer._b.copy_(torch.randint(0, 9, (10,), generator=g).float())
    e = layer._compute_ebops((1, 24))
    e.backward()
    iq, kq, bq = layer.iq.quantizer, layer.kq.quantizer, layer.bq.quantizer
    d = lambda t: t.detach().reshape(-1).to(dev).requires_grad_(t.requires_grad)  # noqa: E731
    fi, bk, bb = d(iq._f), d(kq._b), d(bq._b)
    m_in = _lib.mode_bits('RND', 'WRAP', training=True, round_params=True)
    m_k = _lib.mode_bits('RND', 'SAT_SYM', training=True, round_params=True, kbi=True)
    var = torch.zeros((), dtype=torch.int32, device=dev)
    val, _ = ops.dense_ebops(iq._k.reshape(-1).to(dev), d(iq._i), fi, kq._k.reshape(-1).to(dev), bk,
                             bq._k.to(dev), bb, 1, 24, 10, 1.0, 1.0, 1.0, 10.0, m_in, m_k, m_k, ebops_var=var)
    assert val.item() == e.item() and var.item() == int(e.item())
    val.backward()
    assert torch.equal(fi.grad.cpu(), iq._f.grad.reshape(-1))
    assert torch.equal(bk.grad.cpu(), kq._b.grad.reshape(-1))
    assert torch.equal(bb.grad.cpu(), bq._b.grad.reshape(-1))
    # loss-term form: ebops * beta with the gradient scaled by beta, input integer bits tracked first
    beta = torch.tensor(0.25, device=dev)
    amax = torch.randint(0, 2**30, (7, 24), dtype=torch.int32, device=dev)
    i_track = d(iq._i).clone()
    want_i = i_track.clone()
    ops.wrap_track_i_(amax, want_i, fi.detach(), 0.01, _lib.mode_bits('RND', 'WRAP', training=True))
    with torch.no_grad():
        layer.iq.quantizer._i.copy_(want_i.cpu().reshape(1, 24))
    for v in (iq._f, kq._b, bq._b):
        v.grad = None
    e2 = layer._compute_ebops((1, 24)) * 0.25
    e2.backward()
    fi2, bk2, bb2 = d(iq._f), d(kq._b), d(bq._b)
    _, term = ops.dense_ebops(iq._k.reshape(-1).to(dev), i_track, fi2, kq._k.reshape(-1).to(dev), bk2, bq._k.to(dev), bb2,
                              1, 24, 10, 1.0, 1.0, 1.0, 10.0, m_in, m_k, m_k, amax=amax, decay=0.01, beta=beta, ebops_var=var)
    assert torch.equal(i_track, want_i)
    assert term.item() == e2.item() and var.item() == int(e2.item() / 0.25)
    term.backward()
    assert torch.equal(fi2.grad.cpu(), iq._f.grad.reshape(-1))
    assert torch.equal(bk2.grad.cpu(), kq._b.grad.reshape(-1))
    assert torch.equal(bb2.grad.cpu(), bq._b.grad.reshape(-1))


def test_ebops_scaling_is_a_product_then_a_correctly_rounded_division(dev):
    """``ebops * pf / n_parallel * ebops_factor`` left to right in fp32 (reference src/hgq/layers/core/dense.py:80,
    base.py:102), checked against numpy's IEEE arithmetic: a reciprocal multiply or one precomputed factor lands one ulp
    off for some values, and the uint32 cast of the estimate then one count off (6887 * 121 / 121 is such a case)."""
    _lib, ops = _ops()
    from hgq2_amd.layers.core.base import scale_ebops

    rng = np.random.default_rng(5)
    vals = np.concatenate([[6887.0], rng.integers(1, 2**23, 4000)]).astype(np.float32)
    for pf, n_par in ((121, 121), (7, 49), (3, 1), (25, 36), (1, 3)):
        want = vals * np.float32(pf) / np.float32(n_par)
        got = scale_ebops(torch.from_numpy(vals).to(dev), pf, n_par).cpu().numpy()
        assert np.array_equal(got, want), (pf, n_par)
    # the dense kernel: bits chosen so that the sum is a value a reciprocal multiply gets wrong
    K, N = 71, 97  # sum = 71 * 97 = 6887 for one-bit inputs and one-bit kernels
    m_in = _lib.mode_bits('RND', 'WRAP', training=True, round_params=True)
    m_k = _lib.mode_bits('RND', 'SAT_SYM', training=True, round_params=True, kbi=True)
    k0 = torch.zeros(K, dtype=torch.uint8, device=dev)
    kk = torch.zeros(K * N, dtype=torch.uint8, device=dev)
    for pf, n_par, factor in ((121, 121, 1.0), (7, 49, 0.3), (5, 11, 1.7)):
        i_in = torch.ones(K, device=dev)
        f_in = torch.zeros(K, device=dev, requires_grad=True)
        b_k = torch.ones(K * N, device=dev, requires_grad=True)
        var = torch.zeros((), dtype=torch.int32, device=dev)
        val, _ = ops.dense_ebops(k0, i_in, f_in, kk, b_k, None, None, 1, K, N, pf, n_par, factor, 0.0, m_in, m_k, 0, ebops_var=var)
        want = np.float32(6887.0) * np.float32(pf) / np.float32(n_par) * np.float32(factor)
        assert val.item() == want and var.item() == int(want), (pf, n_par, factor, val.item(), want)
        val.backward()
        g = np.float32(1.0) * np.float32(factor) / np.float32(n_par) * np.float32(pf)  # the chain rule, last operation first
        assert torch.equal(b_k.grad, torch.full_like(b_k, float(g))) and torch.equal(f_in.grad, torch.full_like(f_in, float(g * np.float32(N))))


def test_queued_updates_of_one_quantizer_run_in_turn(dev):
    """Integer-bit updates queued during a model call go out together; the updates of a quantizer that several layers
    share (reference src/hgq/layers/attn/mha.py:205-210) must still be applied one after the other, each from the value the
    previous one left, and the library refuses a launch in which two items update the same variable."""
    import ctypes

    _lib, ops = _ops()
    g = torch.Generator().manual_seed(23)
    m = 200
    mode = _lib.mode_bits('RND', 'WRAP', training=True)
    fb = torch.randint(0, 5, (m,), generator=g).float().to(dev)
    amaxs = [(torch.rand(3, m, generator=g) * s).view(torch.int32).to(dev) for s in (0.5, 8.0, 2.0)]  # bit patterns of |x|
    other_i, other_amax = torch.zeros(m, device=dev), (torch.rand(1, m, generator=g) * 4).view(torch.int32).to(dev)
    start = torch.randint(-2, 6, (m,), generator=g).float().to(dev)
    want = start.clone()
    for a in amaxs:
        ops.wrap_track_i_(a, want, fb, 0.75, mode)
    want_other = other_i.clone()
    ops.wrap_track_i_(other_amax, want_other, fb, 0.75, mode)
    got = start.clone()
    ops.begin_deferred()
    ops.wrap_track_i_(amaxs[0], got, fb, 0.75, mode)
    ops.wrap_track_i_(other_amax, other_i, fb, 0.75, mode)
    ops.wrap_track_i_(amaxs[1], got, fb, 0.75, mode)
    ops.wrap_track_i_(amaxs[2], got, fb, 0.75, mode)
    assert torch.equal(got, start), 'queued, not yet applied'
    ops.end_deferred()
    assert torch.equal(got, want) and torch.equal(other_i, want_other)
    assert not torch.equal(want, start)
    items = (ops._TrackItem * 2)()
    for t in range(2):
        items[t] = ops._TrackItem(amaxs[t].data_ptr(), None, 3, got.data_ptr(), fb.data_ptr(), None, m, 0.75, 0.0, 0.0, mode)
    assert _lib.load().hgq_wrap_track_i_multi(items, 2, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) != 0
    assert torch.equal(got, want), 'a refused call changes nothing'


def test_bias_and_affine_gradients_without_framework_reductions(dev):
    """``bias_add_rows`` / ``affine_rows``: values are the plain tensor expressions; the gradients of the small operands are
    column sums taken by the library's fixed-order reduction (a framework reduction inside a captured step records a
    memory-clearing node, which replays wrongly on this platform)."""
    _lib, ops = _ops()
    g = torch.Generator().manual_seed(41)
    y = torch.randn(1000, 16, 64, generator=g).to(dev)
    up = torch.randn(1000, 16, 64, generator=g).to(dev)
    for b_shape in ((16, 64), (1, 64), (16, 1), (64,)):
        b1 = torch.randn(b_shape, generator=g).to(dev).requires_grad_(True)
        b2 = b1.detach().clone().requires_grad_(True)
        y1, y2 = y.clone().requires_grad_(True), y.clone().requires_grad_(True)
        out = ops.bias_add_rows(y1, b1)
        assert torch.equal(out, y2 + b2)
        (out * up).sum().backward()
        ((y2 + b2).double() * up.double()).sum().backward()
        assert torch.equal(y1.grad, y2.grad)
        scale = up.abs().double().sum(0).sum_to_size(b_shape)
        assert torch.all((b1.grad.double() - b2.grad.double()).abs() <= 1e-6 * scale + 1e-30), b_shape
    x = torch.randn(300, 7, 24, generator=g).to(dev)
    up = torch.randn(300, 7, 24, generator=g).to(dev)
    s1, o1 = torch.randn(1, 1, 24, generator=g).to(dev).requires_grad_(True), torch.randn(1, 1, 24, generator=g).to(dev).requires_grad_(True)
    s2, o2 = s1.detach().double().requires_grad_(True), o1.detach().double().requires_grad_(True)
    x1, x2 = x.clone().requires_grad_(True), x.double().requires_grad_(True)
    out = ops.affine_rows(x1, s1, o1)
    assert torch.equal(out, x * s1.detach() + o1.detach())
    (out * up).sum().backward()
    ((x2 * s2 + o2) * up.double()).sum().backward()
    assert torch.allclose(x1.grad.double(), x2.grad, rtol=1e-6, atol=1e-7)
    assert torch.all((s1.grad.double() - s2.grad).abs() <= 1e-6 * (up.double() * x.double()).abs().sum((0, 1), keepdim=True))
    assert torch.all((o1.grad.double() - o2.grad).abs() <= 1e-6 * up.double().abs().sum((0, 1), keepdim=True))


@pytest.mark.parametrize('rows,K,N,bits_x,bits_w,act', [(4096, 64, 64, 6, 6, 1), (1000, 64, 32, 12, 5, 0), (513, 48, 33, 12, 12, 1),
                                                        (2000, 16, 64, 22, 22, 0), (70, 4, 4, 5, 5, 0), (3000, 20, 12, 8, 16, 1)])
def test_dense_on_bf16_parts_is_the_fp32_contraction(dev, rows, K, N, bits_x, bits_w, act):
    """The streaming dense kernels contract on the bf16 matrix cores after splitting every fp32 operand exactly into up to
    three bf16 parts (8 + 8 + 8 significant bits).  Products of parts are exact and the accumulation is fp32, so the
    result is the fp32 contraction up to the order of the accumulation: against float64 both instructions sit within
    1e-6 of the sum of |terms|, and where every partial sum is exactly representable (few-bit operands) they agree bit
    for bit.  Operands of 5 to 22 bits exercise one, two and three parts on either side."""
    _lib, ops = _ops()
    lib = _lib.load()
    g = torch.Generator().manual_seed(rows + K)
    x = (torch.round(torch.randn(rows, K, generator=g) * 2 ** (bits_x - 3)) / 2 ** (bits_x - 3)).to(dev)
    w = (torch.round(torch.randn(K, N, generator=g) * 2 ** (bits_w - 2)) / 2 ** bits_w).to(dev)
    b = (torch.round(torch.randn(N, generator=g) * 16) / 16).to(dev)
    dy, e = torch.randn(rows, N, generator=g).to(dev), x.new_empty(0)
    want = x.double() @ w.double() + b.double()
    mask = (want > 0).double() if act else torch.ones_like(want)
    want = want * mask
    dz = dy.double() * mask
    refs = (want, dz @ w.double().T, x.double().T @ dz, dz.sum(0))
    scales = (x.double().abs() @ w.double().abs() + b.double().abs(), dz.abs() @ w.double().abs().T, x.double().abs().T @ dz.abs(), dz.abs().sum(0))
    was = lib.hgq_dense_use_bf16_parts(-1)
    got = {}
    try:
        for on in (0, 1):
            lib.hgq_dense_use_bf16_parts(on)
            y, _ = ops.qdense_fwd(x, e, e, e, w, b, act, 0, 0, False)
            dx, dqw, dqb, _ = ops.qdense_bwd(dy, y, x, e, w, True, act, 0, 0)
            got[on] = (y, dx, dqw, dqb)
            for name, t, want_t, sc in zip(('y', 'dx', 'dW', 'db'), got[on], refs, scales):
                err = ((t.double() - want_t).abs() / (sc + 1e-30)).max().item()
                assert err <= 1e-6, f'{name} with bf16 parts = {on}: {err:.2e} of the sum of |terms|'
    finally:
        lib.hgq_dense_use_bf16_parts(was)
    if bits_x + bits_w + 7 <= 24:  # every partial sum of x W is exact in fp32: no accumulation order to differ in
        assert torch.equal(got[0][0], got[1][0])


def test_sparse_ce_and_sgd(dev):
    _lib, ops = _ops()
    g = torch.Generator().manual_seed(17)
    logits = (torch.randn(16384, 5, generator=g) * 3).requires_grad_(True)
    labels = torch.randint(0, 5, (16384,), generator=g)
    loss = torch.nn.functional.cross_entropy(logits.double(), labels)
    loss.backward()
    ld = logits.detach().to(dev).requires_grad_(True)
    got = ops.sparse_ce(ld, labels.to(dev))
    got.backward()
    assert abs(got.item() - loss.item()) <= RTOL * abs(loss.item())
    # d loss / d logit = (softmax - onehot) / rows: a difference of two terms, bounded by 1e-5 of their |sum|
    p64 = torch.softmax(logits.detach().double(), dim=1)
    onehot = torch.nn.functional.one_hot(labels, 5).double()
    want_g, scale_g = (p64 - onehot) / 16384, (p64 + onehot) / 16384
    assert torch.all((ld.grad.cpu().double() - want_g).abs() <= RTOL * scale_g)
    # a label outside [0, C) reads nothing: NaN loss, a zero gradient row, the other rows untouched
    bad = labels.clone()
    bad[5], bad[77] = -1, 5
    lb = logits.detach().to(dev).requires_grad_(True)
    got_bad = ops.sparse_ce(lb, bad.to(dev))
    got_bad.backward()
    assert torch.isnan(got_bad).item()
    gb = lb.grad.cpu()
    assert torch.all(gb[5] == 0) and torch.all(gb[77] == 0)
    keep = torch.ones(16384, dtype=torch.bool)
    keep[5] = keep[77] = False
    assert torch.equal(gb[keep], ld.grad.cpu()[keep])
    # the loss is handed over between workgroups through state words that must be zero again after every call - also
    # after the call with a NaN above -, and the workgroups' sums meet as integers: every run gives the same bits
    for _ in range(20):
        again = ops.sparse_ce(logits.detach().to(dev), labels.to(dev))
        assert again.item() == got.item()
    # without state words one workgroup adds everything up: the same value to rounding, through the C entry point
    lone, dl = torch.empty((), device=dev), torch.empty(16384, 5, device=dev)
    rc = _lib.load().hgq_sparse_ce_fwd_bwd(ld.data_ptr(), labels.to(dev).data_ptr(), lone.data_ptr(), dl.data_ptr(), 16384, 5, None, None)
    assert rc == 0
    assert abs(lone.item() - loss.item()) <= RTOL * abs(loss.item()) and torch.equal(dl, ld.grad)
    w = torch.randn(1000, generator=g) * 10
    gr = torch.randn(1000, generator=g) * 100
    wd = w.to(dev)
    ops.sgd_update_(wd, gr.to(dev), 0.01, 1e-8, -2.0, 2.0)
    assert torch.equal(wd.cpu(), torch.clamp(w - 0.01 * (gr + 1e-8), -2.0, 2.0))
    # many variables in one launch (more than one descriptor batch)
    ws = [torch.randn(n, generator=g) for n in ([5, 1024, 37, 2048] * 15)]
    gs = [torch.randn(t.shape, generator=g) for t in ws]
    wds, gds = [t.to(dev) for t in ws], [t.to(dev) for t in gs]
    n = len(ws)
    ops.sgd_update_multi_(wds, gds, [1e-8] * n, [-1.0] * n, [float('inf')] * n, 0.05)
    for wd_, w_, g_ in zip(wds, ws, gs):
        assert torch.equal(wd_.cpu(), torch.clamp(w_ - 0.05 * (g_ + 1e-8), min=-1.0))
    # loss terms riding along with the update: the same additions in the same order as the launch of their own,
    # the update unchanged
    terms = [(torch.randn((), generator=g) * 10.0 ** (t % 5)).to(dev) for t in range(ops.SUM_BATCH)]
    for n_terms in (1, 3, ops.SUM_BATCH):
        wds2, out = [t.to(dev) for t in ws], torch.full((), float('nan'), device=dev)
        ops.sgd_update_multi_(wds2, gds, [1e-8] * n, [-1.0] * n, [float('inf')] * n, 0.05, sum_terms=terms[:n_terms], sum_out=out)
        assert torch.equal(out, ops.sum_scalars([t.clone() for t in terms[:n_terms]]).reshape(()))
        assert all(torch.equal(a, b) for a, b in zip(wds2, wds))
    with pytest.raises(ValueError):
        ops.sgd_update_multi_(wds2, gds, [0.0] * n, [-1.0] * n, [1.0] * n, 0.05, sum_terms=terms + terms[:1], sum_out=out)


@pytest.mark.parametrize('rows,M', [(4096, 16), (2048, 4096), (1000, 7)])
def test_per_column_bit_width_gradients_have_a_fixed_order(dev, rows, M):
    """Bit-widths shared along the leading axis: the reduced gradients come from per-chunk slices added in a fixed
    order (hgq_quantize_bwd_sliced), so two runs give the same bits; the value is that of fp64 within fp32 rounding."""
    _lib, ops = _ops()
    g = torch.Generator().manual_seed(rows + M)
    x = (torch.randn(rows, M, generator=g) * 3).to(dev)
    dy = torch.randn(rows, M, generator=g).to(dev)
    k = torch.ones(M, dtype=torch.uint8).to(dev)
    i = torch.randint(1, 4, (M,), generator=g).float().to(dev)
    f = torch.randint(1, 6, (M,), generator=g).float().to(dev)
    mode = _lib.mode_bits('RND', 'WRAP', training=True)
    assert _lib.load().hgq_quantize_bwd_workspace(rows * M, M, 1) > 0
    runs = [ops.quantize_bwd(dy, x, k, i, f, mode, 1, True, False) for _ in range(2)]
    assert torch.equal(runs[0][2], runs[1][2]) and torch.equal(runs[0][0], runs[1][0])
    xq = torch.floor(x.double() * 2.0**f.double() + 0.5) / 2.0**f.double()
    want = (-0.6931471805599453 * (xq - x.double()) * dy.double()).sum(0)
    err = float((runs[0][2].double() - want).abs().max())
    assert err <= 1e-5 * float(want.abs().max()) + 1e-6
    assert torch.equal(runs[0][0], dy)  # straight-through


@pytest.mark.parametrize('shape', [(5, 64), (2, 1024), (2, 63), (300, 7)])
def test_trackers_ignore_the_padding_of_a_row_chunk(dev, shape):
    """A saturating quantizer whose range excludes zero (2**i < 2**-f) maps the zeros that pad a workgroup's row
    chunk to its upper bound; those must not show up in the abs-max / any-negative trackers."""
    _lib, ops = _ops()
    rows, M = shape
    g = torch.Generator().manual_seed(rows)
    x = torch.rand(shape, generator=g) * 0.01  # everything saturates at the (negative) upper bound or at zero
    k = torch.zeros(M)
    k[::2] = 1.0
    i = torch.full((M,), -2.0)
    f = torch.zeros(M)
    for om in ('SAT', 'SAT_SYM'):
        want = ofp.get_fixed_quantizer('RND', om)(x, *(torch.broadcast_to(t, shape) for t in (k, i, f)), True, None)
        mode = _lib.mode_bits('RND', om, training=True)
        y, amax, neg = ops.quantize(x.to(dev), k.to(dev), i.to(dev), f.to(dev), mode, bw_inner=1, track=True)
        assert torch.equal(y.cpu(), want)
        amax, neg = amax.view(-1, M).amax(0), neg.view(-1, M).amax(0)
        assert torch.equal(amax.view(torch.float32).cpu(), want.abs().amax(0))
        assert torch.equal(neg.cpu(), (want < 0).int().amax(0))


def _dense_sweep_cases(n, seed=0):
    import random

    rnd = random.Random(seed)
    cases = []
    for _ in range(n):
        K = rnd.choice([4, 8, 12, 16, 20, 32, 36, 48, 64])
        N = rnd.choice([1, 3, 4, 5, 8, 10, 16, 24, 31, 32, 33, 40, 64])
        P = rnd.choice([0, 1, 2, 4, 8, 16, 32, 64])
        rows = rnd.choice([1, 7, 63, 64, 65, 200, 640, 1000]) * (P or 1)
        cases.append((rows, K, N, P, rnd.choice([0, 1]), rnd.choice([True, False]), rnd.choice(ROUND)))
    return cases


@pytest.mark.parametrize('rows,K,N,P,act,has_bias,round_mode', _dense_sweep_cases(40))
def test_qdense_sweep_against_fp64(dev, rows, K, N, P, act, has_bias, round_mode):
    """ops.qdense over widths that are and are not multiples of 4 / 32, table heights 0 (no input quantizer) to 64, ragged
    last tiles: output, abs-max slices, dx, dW, db and the fractional-bit gradient against an fp64 statement."""
    _lib, ops = _ops()
    g = torch.Generator().manual_seed(rows * 131 + K * 7 + N)
    x = torch.randn(rows, K, generator=g) * 2
    w = torch.randn(K, N, generator=g) * 0.4
    b = torch.randn(N, generator=g) if has_bias else None
    up = torch.randn(rows, N, generator=g)
    if P:
        f = torch.randint(1, 6, (P, K), generator=g).float()
        fr = f.repeat(rows // P, 1)
        t = x * 2.0**fr
        xq = (torch.floor(t + 0.5) if round_mode == 'RND' else torch.floor(t) if round_mode == 'TRN' else torch.round(t)) / 2.0**fr
    else:
        xq = x
    xr, wr = xq.double().requires_grad_(True), w.double().requires_grad_(True)
    br = b.double().requires_grad_(True) if has_bias else None
    z = xr @ wr + (br if has_bias else 0)
    if act:  # no upstream gradient where fp32 and fp64 may disagree on the side of the kink
        up = up * (z.detach().abs() > 1e-5 * float(z.detach().abs().max())).float()
    y_r = torch.relu(z) if act else z
    (y_r * up.double()).sum().backward()
    xd, wd = x.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
    bd = b.to(dev).requires_grad_(True) if has_bias else None
    if P:
        fd = f.to(dev).requires_grad_(True)
        mode = _lib.mode_bits(round_mode, 'WRAP', training=True, round_params=True)
        kk, ii = torch.ones(P * K, dtype=torch.uint8, device=dev), torch.full((P * K,), 3.0, device=dev)
        y, amax = ops.qdense(xd, kk, ii, fd.view(-1), wd, bd, act, mode, P, True)
        am = amax.view(-1, P * K).amax(0).view(torch.float32).cpu().view(P, K)
        assert torch.equal(am, xq.abs().view(rows // P, P, K).amax(0))
    else:
        y, _ = ops.qdense(xd, None, None, None, wd, bd, act, 0, 0, False)
    (y * up.to(dev)).sum().backward()
    checks = [('y', y.detach(), y_r.detach()), ('dx', xd.grad, xr.grad), ('dw', wd.grad, wr.grad)]
    if has_bias:
        checks.append(('db', bd.grad, br.grad))
    if P:
        df_r = (-np.log(2) * (xq.double() - x.double()) * xr.grad).view(rows // P, P, K).sum(0)
        checks.append(('df', fd.grad.view(P, K), df_r))
    # bounds: 1e-5 of the sum of the |products| behind every entry - the same contraction on the absolute values
    dz = (up.double() * (z.detach() > 0)) if act else up.double()
    xa, wa = xq.double().abs(), w.double().abs()
    scales = {'y': xa @ wa + (b.double().abs() if has_bias else 0), 'dx': dz.abs() @ wa.T, 'dw': xa.T @ dz.abs(), 'db': dz.abs().sum(0)}
    if P:
        scales['df'] = (np.log(2) * (xq.double() - x.double()).abs() * (dz.abs() @ wa.T)).view(rows // P, P, K).sum(0)
    for name, got, want in checks:
        err = (got.cpu().double() - want.double()).abs()
        tol = RTOL * scales[name] + 1e-30
        assert bool((err <= tol).all()), f'{name}: {float((err / tol).max()):.2f} x the bound of 1e-5 of the summed |terms|'


@pytest.mark.parametrize('K,N,overflow', [(16, 64, 'SAT_SYM'), (64, 32, 'SAT'), (5, 7, 'SAT_SYM'), (130, 20, 'SAT')])
def test_bn_fold_with_its_quantizers_in_one_launch(dev, K, N, overflow):
    """`bn_fold_quant` = `bn_fold` followed by the kernel and bias quantizers (reference
    src/hgq/layers/einsum_dense_batchnorm.py:158-211): the quantized values and the moving statistics equal the separate
    launches' bit for bit (the same arithmetic per element), every gradient to the order of the column sums."""
    _lib, ops = _ops()
    g = torch.Generator().manual_seed(K * N)
    mode = _lib.mode_bits('RND', overflow, training=True, kbi=True, round_params=True)
    mk = lambda *s, scale=1.0: (torch.randn(*s, generator=g) * scale).to(dev)  # noqa: E731
    w, bias, gamma, mean = mk(K, N, scale=0.5), mk(N), mk(N).abs() + 0.5, mk(N, scale=0.3)
    meansq = mean * mean + mk(N).abs() * 0.5 + 0.01
    qk = (torch.ones(K * N, dtype=torch.uint8, device=dev), torch.randint(0, 3, (K * N,), generator=g).float().to(dev),
          (torch.randint(2, 9, (K * N,), generator=g).float() + torch.rand(K * N, generator=g) * 0.4).to(dev))
    qb = (torch.ones(N, dtype=torch.uint8, device=dev), torch.randint(0, 3, (N,), generator=g).float().to(dev),
          (torch.randint(2, 9, (N,), generator=g).float() + torch.rand(N, generator=g) * 0.4).to(dev))
    up_w, up_b = mk(K, N), mk(N)

    def run(fused):
        leaves = [t.clone().requires_grad_(True) for t in (w, bias, gamma, mean, meansq, qk[1], qk[2], qb[1], qb[2])]
        lw, lb, lg, lm, ls, ik, fk, ib, fb = leaves
        mm, mv = torch.zeros(N, device=dev), torch.ones(N, device=dev)
        if fused:
            qw, qbias = ops.bn_fold_quant(lw, lb, lg, lm, ls, True, 1e-3, mm, mv, 0.9, (qk[0], ik, fk, mode), (qb[0], ib, fb, mode))
        else:
            fw, fbias = ops.bn_fold(lw, lb, lg, lm, ls, True, 1e-3, mm, mv, 0.9)
            qw, qbias = ops.quantize_multi([fw, fbias], [qk[0], qb[0]], [ik, ib], [fk, fb], [mode, mode])
        ((qw * up_w).sum() + (qbias * up_b).sum()).backward()
        return (qw.detach(), qbias.detach(), mm, mv), [t.grad for t in leaves]

    (vals_a, grads_a), (vals_b, grads_b) = run(True), run(False)
    for a, b in zip(vals_a, vals_b):
        assert torch.equal(a, b)
    for name, a, b in zip(('w', 'bias', 'gamma', 'mean', 'meansq', 'i_k', 'b_k', 'i_b', 'b_b'), grads_a, grads_b):
        assert (a is None) == (b is None), name
        if a is not None:
            err = (a.double() - b.double()).abs().max().item()
            assert err <= 1e-5 * (b.abs().max().item() + 1e-6), (name, err)


@pytest.mark.parametrize('R,G,K,N,act,bias', [(300, 5, 7, 9, 1, True), (1, 1, 1, 1, 0, False), (4096, 3, 16, 16, 1, True), (70, 12, 64, 64, 0, True),
                                              (65, 2, 33, 5, 1, False), (100000, 4, 8, 8, 0, True), (0, 3, 4, 4, 0, True)])
def test_grouped_dense_against_fp64(dev, R, G, K, N, act, bias):
    """``y[r, g] = act(x[r, g] @ w[g] + b[g])`` (the einsum 'Babc,bcd->Babd' of reference tests/test_dense.py:56 on
    [rows, groups, in] views): values and all three gradients within 1e-5 of the summed |terms| of a float64 einsum."""
    _lib, ops = _ops()
    g = torch.Generator().manual_seed(R + 31 * G + K)
    x = torch.randn(R, G, K, generator=g)
    w = torch.randn(G, K, N, generator=g) * 0.4
    b = torch.randn(G, N, generator=g) if bias else None
    up = torch.randn(R, G, N, generator=g)
    xr, wr = x.double().requires_grad_(True), w.double().requires_grad_(True)
    br = b.double().requires_grad_(True) if bias else None
    z = torch.einsum('rgk,gkn->rgn', xr, wr) + (br if bias else 0)
    if act:  # no upstream gradient where fp32 and fp64 may disagree on the side of the kink
        up = up * (z.detach().abs() > 1e-5 * float(z.detach().abs().max() if R else 1)).float()
    yr = torch.relu(z) if act else z
    (yr * up.double()).sum().backward()
    xd, wd = x.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
    bd = b.to(dev).requires_grad_(True) if bias else None
    assert ops.gdense_supported(xd, wd)
    y = ops.gdense(xd, wd, bd, act)
    assert tuple(y.shape) == (R, G, N)
    (y * up.to(dev)).sum().backward()
    dz = (up.double() * (z.detach() > 0)) if act else up.double()
    xa, wa = x.double().abs(), w.double().abs()
    scales = {'y': torch.einsum('rgk,gkn->rgn', xa, wa) + (b.double().abs() if bias else 0),
              'dx': torch.einsum('rgn,gkn->rgk', dz.abs(), wa), 'dw': torch.einsum('rgk,rgn->gkn', xa, dz.abs()), 'db': dz.abs().sum(0)}
    checks = [('y', y.detach(), yr.detach()), ('dx', xd.grad, xr.grad), ('dw', wd.grad, wr.grad)] + ([('db', bd.grad, br.grad)] if bias else [])
    for name, got, want in checks:
        err = (got.cpu().double() - want).abs()
        tol = RTOL * scales[name] + 1e-30
        assert bool((err <= tol).all()), f'{name}: {float((err / tol).max()):.2f} x the bound'


@pytest.mark.parametrize('shape', [(1000, 64), (7, 3, 5, 8), (1, 4), (100000, 12), (0, 16)])
def test_affine_rows_against_fp64(dev, shape):
    """``x * s + o`` over the trailing channel axis (QBatchNormalization's map): values exactly the two fp32 operations,
    dx exactly, the two parameter gradients within 1e-5 of the summed |terms|."""
    _lib, ops = _ops()
    g = torch.Generator().manual_seed(sum(shape))
    C = shape[-1]
    x, up = torch.randn(shape, generator=g), torch.randn(shape, generator=g)
    s, o = torch.randn(C, generator=g), torch.randn(C, generator=g)
    xd, sd, od = (t.to(dev).requires_grad_(True) for t in (x, s, o))
    if x.numel() == 0:
        return  # the layer does not call the kernels on empty inputs
    y = ops.affine_rows(xd, sd, od)
    assert y.grad_fn is not None and type(y.grad_fn).__name__.startswith('_AffineRows')
    assert torch.equal(y.detach().cpu(), x * s + o)
    y.backward(up.to(dev))
    assert torch.equal(xd.grad.cpu(), up * s)
    rows = x.reshape(-1, C).double()
    u2 = up.reshape(-1, C).double()
    for got, terms, name in ((sd.grad, u2 * rows, 'dscale'), (od.grad, u2, 'doffset')):
        _assert_close_sum(got, terms.sum(0), terms.abs().sum(0), name)
