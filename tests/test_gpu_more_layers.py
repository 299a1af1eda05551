"""GPU parity of QEinsumDense, QEinsumDenseBatchnorm, QUnaryFunctionLUT / QSoftmax,
QMultiHeadAttention and QConv2D against the CPU oracle twins (same weights, bit-widths, inputs):
forward values, the loss terms, state updates, and the gradients of every trainable variable."""

import pytest
import torch

from oracle import twin

pytestmark = pytest.mark.gpu
RTOL = 1e-5


class Scopes:
    def __init__(self, *scopes):
        self.scopes = scopes

    def __enter__(self):
        for s in self.scopes:
            s.__enter__()

    def __exit__(self, *a):
        for s in reversed(self.scopes):
            s.__exit__(*a)


def readme_scopes(beta0=1e-5):
    from hgq2_amd.config import LayerConfigScope, QuantizerConfigScope

    return Scopes(QuantizerConfigScope(place='all', default_q_type='kbi', overflow_mode='SAT_SYM'),
                  QuantizerConfigScope(place='datalane', default_q_type='kif', overflow_mode='WRAP'),
                  LayerConfigScope(enable_ebops=True, beta0=beta0))


def _close(got, want, rtol=RTOL, floor=1e-6, what=''):
    got, want = got.detach().double().cpu(), want.detach().double()
    tol = rtol * (want.abs().max() + floor) + rtol * want.abs()
    err = (got - want).abs()
    assert torch.all(err <= tol), f'{what}: max err {err.max():.3e} (tol {tol.max():.3e})'


def _perturb(layer, g):
    """Randomise bit-widths a little so they are heterogeneous (reference tests/base.py:161-182)."""
    from hgq2_amd.quantizer.internal import FixedPointQuantizerKBI, FixedPointQuantizerKIF

    with torch.no_grad():
        for m in layer.modules():
            if isinstance(m, FixedPointQuantizerKBI):
                m._b.copy_(torch.randint(3, 9, m._b.shape, generator=g).float())
            elif isinstance(m, FixedPointQuantizerKIF):
                m._f.copy_(torch.randint(3, 8, m._f.shape, generator=g).float())


def _compare_step(layer, ref_layer, run_prod, run_ref, named_prod, named_ref, grad_rtol=RTOL):
    """One training forward+backward on both sides; compares output, loss terms and gradients."""
    from hgq2_amd.train import model_loss
    from oracle import hgq_ref

    out_p = run_prod(True)
    loss_p = model_loss(layer, (out_p * out_p).mean())
    loss_p.backward()
    # the oracle's contractions run in float64 (its quantizers stay fp32): the bound then measures the kernels, not the
    # fp32 summation order of the CPU restatement
    hgq_ref.ACC64 = True
    try:
        out_r = run_ref(True)
        loss_r = (out_r * out_r).mean() + ref_layer.extra_loss()
        loss_r.backward()
    finally:
        hgq_ref.ACC64 = False
    _close(out_p, out_r, what='output')
    assert abs(loss_p.item() - loss_r.item()) <= RTOL * abs(loss_r.item()) + 1e-9
    for (name, p), (_, r) in zip(named_prod, named_ref):
        if r.grad is None:
            assert p.grad is None or float(p.grad.abs().max()) == 0.0, name
            continue
        assert p.grad is not None, f'{name} has no gradient'
        _close(p.grad, r.grad, rtol=grad_rtol, floor=1e-9, what=f'grad {name}')


def test_einsum_dense_gemm_forms(dev):
    from hgq2_amd.layers import QEinsumDense

    g = torch.Generator().manual_seed(0)
    for eq, in_shape, out_shape, bias_axes in [('bpf,fh->bph', (64, 12, 16), (12, 24), 'h'),
                                                ('abc,cde->abde', (32, 10, 16), (10, 4, 8), 'de'),
                                                ('abcd,cde->abe', (32, 10, 4, 8), (10, 16), 'e'),
                                                ('Bij,ijk->Bik', (50, 3, 4), (3, 6), 'ik')]:
        with readme_scopes():
            layer = QEinsumDense(eq, out_shape, bias_axes=bias_axes, activation='relu')
        x = (torch.randn(in_shape, generator=g) * 2)
        layer(x.to(dev), training=True)  # build + adapt integer bits
        _perturb(layer, g)
        with torch.no_grad():
            layer.bias.copy_(torch.randn(layer.bias.shape, generator=g) * 0.3)
        r = twin.ref_einsum_dense(layer, in_shape)
        xp = x.to(dev).requires_grad_(True)
        xr = x.clone().requires_grad_(True)
        named_p = [('x', xp), ('kernel', layer._kernel), ('bias', layer.bias), ('iq_f', layer.iq.quantizer._f),
                   ('kq_b', layer.kq.quantizer._b), ('kq_i', layer.kq.quantizer._i), ('bq_b', layer.bq.quantizer._b)]
        named_r = [('x', xr), ('kernel', r.kernel), ('bias', r.bias), ('iq_f', r.iq.quantizer._f),
                   ('kq_b', r.kq.quantizer._b), ('kq_i', r.kq.quantizer._i), ('bq_b', r.bq.quantizer._b)]
        _compare_step(layer, r, lambda t: layer(xp, training=t), lambda t: r(xr, training=t), named_p, named_r)
        assert torch.equal(layer.iq.quantizer._i.cpu(), r.iq.quantizer._i.detach()), eq
        assert int(layer.ebops.cpu().view(torch.int32)) == int(r.ebops_value), eq


def test_einsum_dense_batchnorm(dev):
    from hgq2_amd.layers import QEinsumDenseBatchnorm

    g = torch.Generator().manual_seed(1)
    with readme_scopes():
        layer = QEinsumDenseBatchnorm('bpf,fh->bph', (16, 32), bias_axes='h', activation='relu')
    x = torch.randn(128, 16, 16, generator=g)
    layer(x.to(dev), training=True)
    _perturb(layer, g)
    r = twin.ref_einsum_dense_bn(layer, tuple(x.shape))
    xp, xr = x.to(dev).requires_grad_(True), x.clone().requires_grad_(True)
    named_p = [('x', xp), ('kernel', layer._kernel), ('bias', layer.bias), ('gamma', layer.bn_gamma),
               ('iq_f', layer.iq.quantizer._f), ('kq_b', layer.kq.quantizer._b)]
    named_r = [('x', xr), ('kernel', r.kernel), ('bias', r.bias), ('gamma', r.gamma), ('iq_f', r.iq.quantizer._f),
               ('kq_b', r.kq.quantizer._b)]
    _compare_step(layer, r, lambda t: layer(xp, training=t), lambda t: r(xr, training=t), named_p, named_r)
    _close(layer.moving_mean, r.moving_mean, what='moving_mean')
    _close(layer.moving_variance, r.moving_variance, what='moving_variance')
    with torch.no_grad():
        _close(layer(x.to(dev), training=False), r(x, training=False), what='inference output')


def test_softmax_table_pipeline(dev):
    from hgq2_amd.config import QuantizerConfig
    from hgq2_amd.layers import QSoftmax

    g = torch.Generator().manual_seed(2)
    with readme_scopes():
        layer = QSoftmax(axis=-1, enable_oq=True, exp_iq_conf=QuantizerConfig(place='datalane', overflow_mode='SAT'),
                         input_scaler=0.25)
    x = torch.randn(64, 4, 16, 16, generator=g) * 3
    layer(x.to(dev), training=True)
    r = twin.ref_softmax(layer)
    xp, xr = x.to(dev).requires_grad_(True), x.clone().requires_grad_(True)
    e, i = layer.exp_table, layer.inv_table
    named_p = [('x', xp), ('exp_iq_f', e.iq.quantizer._f), ('exp_iq_i', e.iq.quantizer._i), ('exp_oq_b', e.oq.quantizer._b),
               ('inv_iq_f', i.iq.quantizer._f), ('inv_oq_b', i.oq.quantizer._b), ('oq_f', layer.oq.quantizer._f)]
    re_, ri = r.exp_table, r.inv_table
    named_r = [('x', xr), ('exp_iq_f', re_.iq.quantizer._f), ('exp_iq_i', re_.iq.quantizer._i),
               ('exp_oq_b', re_.oq.quantizer._b), ('inv_iq_f', ri.iq.quantizer._f), ('inv_oq_b', ri.oq.quantizer._b),
               ('oq_f', r.oq.quantizer._f)]
    _compare_step(layer, r, lambda t: layer(xp, training=t), lambda t: r(xr, training=t), named_p, named_r)
    # with dummy quantizers the layer is the textbook softmax (reference tests/test_activation.py:58-74)
    from hgq2_amd.config import QuantizerConfigScope

    with QuantizerConfigScope(default_q_type='dummy'):
        plain = QSoftmax(axis=-1, enable_ebops=False)
    y = plain(x.to(dev), training=False)
    assert torch.allclose(y.cpu(), torch.softmax(x, -1), atol=1e-6)


def test_multi_head_attention(dev):
    from hgq2_amd.layers import QMultiHeadAttention

    g = torch.Generator().manual_seed(3)
    for fuse in ('none', 'qkv'):
        with readme_scopes():
            layer = QMultiHeadAttention(num_heads=2, key_dim=8, fuse=fuse)
        x = torch.randn(64, 12, 16, generator=g).clamp(-1, 1)
        layer(x.to(dev), training=True)
        _perturb(layer, g)
        r = twin.ref_mha(layer, tuple(x.shape))
        xp, xr = x.to(dev).requires_grad_(True), x.clone().requires_grad_(True)
        named_p = [('x', xp), ('wq', layer._query_dense._kernel), ('wk', layer._key_dense._kernel),
                   ('wv', layer._value_dense._kernel), ('wo', layer._output_dense._kernel),
                   ('q_oq_f', layer._query_dense.oq.quantizer._f), ('sm_oq_f', layer._softmax.oq.quantizer._f),
                   ('v_iq_f', layer._value_dense.iq.quantizer._f)]
        named_r = [('x', xr), ('wq', r.qd.kernel), ('wk', r.kd.kernel), ('wv', r.vd.kernel), ('wo', r.od.kernel),
                   ('q_oq_f', r.qd.oq.quantizer._f), ('sm_oq_f', r.softmax.oq.quantizer._f), ('v_iq_f', r.vd.iq.quantizer._f)]
        _compare_step(layer, r, lambda t: layer(xp, training=t), lambda t: r(xr, training=t), named_p, named_r)
        assert int(layer._ebops.cpu().view(torch.int32)) == int(r.ebops_value), fuse


@pytest.mark.parametrize('fuse,shapes,causal', [('none', ((2, 4, 8), (2, 4, 9), (2, 4, 10)), False), ('kv', ((2, 4, 3), (2, 4, 5)), False),
                                                ('none', ((3, 2, 8), (2, 5, 6)), False), ('qkv', ((9, 8),), True),
                                                # sequence lengths the one-pass kernels take: the causal rule is applied inside them
                                                ('none', ((32, 16),), True), ('qkv', ((64, 16),), True)])
@pytest.mark.parametrize('num_heads', [1, 2])
def test_multi_head_attention_shapes_of_the_reference_tests(dev, fuse, shapes, causal, num_heads):
    """The input shapes reference tests/test_mha.py:29-37 runs: two sequence axes with separate query / value / key
    inputs of different widths, fused key-value input, and one sequence axis with the causal mask."""
    from hgq2_amd.layers import QMultiHeadAttention

    g = torch.Generator().manual_seed(5 + num_heads)
    B = 48
    with readme_scopes():
        layer = QMultiHeadAttention(num_heads=num_heads, key_dim=8, fuse=fuse)
    xs = [torch.randn((B,) + sh, generator=g).clamp(-1, 1) for sh in shapes]
    kw = {'use_causal_mask': True} if causal else {}
    layer(*[x.to(dev) for x in xs], training=True, **kw)
    _perturb(layer, g)
    r = twin.ref_mha(layer, *[tuple(x.shape) for x in xs])
    xp = [x.to(dev).requires_grad_(True) for x in xs]
    xr = [x.clone().requires_grad_(True) for x in xs]
    mask = torch.tril(torch.ones(1, shapes[0][0], shapes[0][0], dtype=torch.bool)) if causal else None
    named_p = [(f'x{j}', t) for j, t in enumerate(xp)] + [
        ('wq', layer._query_dense._kernel), ('wk', layer._key_dense._kernel), ('wv', layer._value_dense._kernel),
        ('wo', layer._output_dense._kernel), ('q_oq_f', layer._query_dense.oq.quantizer._f), ('k_oq_f', layer._key_dense.oq.quantizer._f),
        ('sm_oq_f', layer._softmax.oq.quantizer._f), ('v_iq_f', layer._value_dense.iq.quantizer._f)]
    named_r = [(f'x{j}', t) for j, t in enumerate(xr)] + [
        ('wq', r.qd.kernel), ('wk', r.kd.kernel), ('wv', r.vd.kernel), ('wo', r.od.kernel), ('q_oq_f', r.qd.oq.quantizer._f),
        ('k_oq_f', r.kd.oq.quantizer._f), ('sm_oq_f', r.softmax.oq.quantizer._f), ('v_iq_f', r.vd.iq.quantizer._f)]
    _compare_step(layer, r, lambda t: layer(*xp, training=t, **kw), lambda t: r(*xr, training=t, mask=mask), named_p, named_r)
    assert int(layer._ebops.cpu().view(torch.int32)) == int(r.ebops_value)
    assert torch.equal(layer._softmax.oq.quantizer._i.cpu(), r.softmax.oq.quantizer._i.detach())
    with torch.no_grad():
        _close(layer(*[x.to(dev) for x in xs], training=False, **kw), r(*xs, training=False, mask=mask), what='inference output')


def test_conv2d_stack_layer(dev):
    from hgq2_amd.layers import QConv2D

    g = torch.Generator().manual_seed(4)
    for padding, strides in (('valid', (1, 1)), ('same', (2, 1))):
        with readme_scopes():
            layer = QConv2D(8, (3, 3), strides=strides, padding=padding, activation='relu')
        x = torch.rand(32, 10, 9, 3, generator=g)
        layer(x.to(dev), training=True)
        _perturb(layer, g)
        r = twin.ref_conv2d(layer)
        xp, xr = x.to(dev).requires_grad_(True), x.clone().requires_grad_(True)
        named_p = [('x', xp), ('kernel', layer._kernel), ('bias', layer.bias), ('iq_f', layer.iq.quantizer._f),
                   ('kq_b', layer.kq.quantizer._b), ('kq_i', layer.kq.quantizer._i)]
        named_r = [('x', xr), ('kernel', r.kernel), ('bias', r.bias), ('iq_f', r.iq.quantizer._f), ('kq_b', r.kq.quantizer._b),
                   ('kq_i', r.kq.quantizer._i)]
        _compare_step(layer, r, lambda t: layer(xp, training=t), lambda t: r(xr, training=t), named_p, named_r)
        assert torch.equal(layer.iq.quantizer._i.cpu(), r.iq.quantizer._i.detach())
        assert int(layer.ebops.cpu().view(torch.int32)) == int(r.ebops_value)


def test_einsum_dense_many_tracker_slices(dev):
    """A projection of the attention configuration's size: the fused input quantizer produces more
    abs-max slices than the EBOPs kernel folds in, so the integer bits are tracked by the separate
    kernel over all slices; output, EBOPs and tracked bits must still match the oracle."""
    from hgq2_amd.layers import QEinsumDense
    from hgq2_amd.layers.core import _contraction

    g = torch.Generator().manual_seed(7)
    with readme_scopes():
        layer = QEinsumDense('abc,cde->abde', (64, 4, 16), bias_axes='de')
    x = torch.randn(1024, 64, 64, generator=g) * 2
    layer(x.to(dev), training=True)
    r = twin.ref_einsum_dense(layer, tuple(x.shape))
    from hgq2_amd import _lib

    n_parts = _lib.load().hgq_qdense_fwd_parts(x.shape[0] * x.shape[1])
    assert n_parts * 64 * 64 > _contraction.FUSED_TRACK_MAX
    with torch.no_grad():
        got = layer(x.to(dev), training=True)
        want = r(x, training=True)
    _close(got, want, what='output')
    assert torch.equal(layer.iq.quantizer._i.cpu(), r.iq.quantizer._i.detach())
    assert int(layer.ebops.cpu().view(torch.int32)) == int(r.ebops_value)


@pytest.mark.parametrize('dims', [(8, 64, 64, 4, 16), (5, 12, 20, 2, 8), (3, 33, 7, 3, 40), (2, 64, 64, 1, 64)])
def test_attention_contractions_match_einsum(dev, dims):
    """hgq_attn_scores / hgq_attn_combine and their gradients against the einsum strings they replace (fp64)."""
    from hgq2_amd import ops

    B, T, S, N, H = dims
    g = torch.Generator().manual_seed(B * 100 + T)
    q, k, v = (torch.randn(B, L, N, H, generator=g) for L in (T, S, S))
    p = torch.rand(B, N, T, S, generator=g)
    refs = [t.double().requires_grad_(True) for t in (q, k, v, p)]
    outs = [t.to(dev).requires_grad_(True) for t in (q, k, v, p)]
    want_s = torch.einsum('aecd,abcd->acbe', refs[1], refs[0])
    want_o = torch.einsum('acbe,aecd->abcd', refs[3], refs[2])
    got_s = ops.attn_scores(outs[0], outs[1])
    got_o = ops.attn_combine(outs[3], outs[2])
    us, uo = torch.randn(want_s.shape, generator=g), torch.randn(want_o.shape, generator=g)
    ((want_s * us.double()).sum() + (want_o * uo.double()).sum()).backward()
    ((got_s * us.to(dev)).sum() + (got_o * uo.to(dev)).sum()).backward()
    for name, a, b in [('scores', got_s, want_s), ('out', got_o, want_o)] + [
            (f'grad {n}', o.grad, r.grad) for n, o, r in zip('qkvp', outs, refs)]:
        scale = b.abs().max().item() + 1e-9
        err = float((a.detach().cpu().double() - b.detach()).abs().max())
        assert err <= 1e-5 * scale, f'{name}: {err:.3e} vs scale {scale:.3e}'


@pytest.mark.parametrize('kind', ['conv', 'particle', 'mha'])
def test_graph_replay_equals_eager_steps(dev, kind):
    """A HIP-graph capture of the whole training step (forward, loss, backward, SGD) of the
    convolution, per-particle and attention models, replayed several times with host work and
    synchronisations in between, follows the eager trajectory."""
    from hgq2_amd import ops
    from hgq2_amd.train import SGD, GraphedTrainStep, model_loss
    from hgq2_amd.utils import models

    g = torch.Generator().manual_seed(21)
    if kind == 'conv':
        make = lambda: models.conv_stack(filters=8, n_out=10, device=dev)  # noqa: E731
        xs = [torch.rand(32, 12, 12, 1, generator=g).to(dev) for _ in range(4)]
        ys = [torch.randint(0, 10, (32,), generator=g).to(dev) for _ in range(4)]
        loss_fn = ops.sparse_ce
    elif kind == 'particle':
        make = lambda: models.particle_mlp(n_particles=8, n_features=16, hidden=(32, 16), device=dev)  # noqa: E731
        xs = [torch.randn(64, 8, 16, generator=g).to(dev) for _ in range(4)]
        ys = [torch.randint(0, 5, (64,), generator=g).to(dev) for _ in range(4)]
        loss_fn = ops.sparse_ce
    else:
        make = lambda: models.mha_block(num_heads=2, key_dim=8, device=dev)  # noqa: E731
        xs = [torch.randn(16, 12, 16, generator=g).to(dev) for _ in range(4)]
        ys = [torch.randn(16, 12, 16, generator=g).to(dev) for _ in range(4)]
        loss_fn = lambda out, y: ((out - y) ** 2).mean()  # noqa: E731
    eager, graphed = make(), make()
    eager(xs[0], training=True), graphed(xs[0], training=True)  # build
    graphed.load_state_dict(eager.state_dict())
    opt = SGD(eager.parameters(), lr=0.01, fold_regularizers=True)
    gopt = SGD(graphed.parameters(), lr=0.01, fold_regularizers=True)

    def eager_step(x, y):
        # the step as the captured one runs it: EBOPs launches on the second stream, gradient pieces through the sink
        opt.zero_grad()
        with ops.overlap_ebops():
            loss = model_loss(eager, loss_fn(eager(x, training=True), y), True)
            opt.backward(loss)
            opt.step()
        return loss.detach()

    warm = 3
    for _ in range(warm + 1):
        eager_step(xs[0], ys[0])
    step = GraphedTrainStep(graphed, loss_fn, gopt, xs[0], ys[0], warmup=warm)
    step()
    for x, y in zip(xs[1:], ys[1:]):
        le = eager_step(x, y)
        lg = step(x, y)
        torch.cuda.synchronize()
        # the same launches in the same order on the same numbers: bit for bit
        assert lg.item() == le.item(), kind
        for (name, pe), (_, pg) in zip(eager.state_dict().items(), graphed.state_dict().items()):
            assert torch.equal(pg, pe), f'{kind}: {name}'


def test_graph_replays_with_row_broadcast_parameters(dev):
    """A bias with one value per (position, channel) and the scale / offset of QBatchNormalization get their gradients from
    sums over the batch.  Taken by framework reductions these were right in the first replay of a captured step and wrong
    in later ones (memory-clearing nodes); taken by the library's slice reduction every replay follows the eager step."""
    from hgq2_amd import ops
    from hgq2_amd.core import Sequential
    from hgq2_amd.layers import QBatchNormalization, QEinsumDense
    from hgq2_amd.train import SGD, GraphedTrainStep, model_loss

    g = torch.Generator().manual_seed(22116)
    x = (torch.round(torch.randn(1000, 16, 8, generator=g).clamp(-5, 5) * 256) / 256).to(dev)

    def make():
        torch.manual_seed(5)
        with readme_scopes(beta0=1e-4):
            return Sequential([QEinsumDense('bpf,fh->bph', (16, 64), bias_axes='ph'), QBatchNormalization()])

    eager, graphed = make(), make()
    eager(x, training=True), graphed(x, training=True)
    graphed.load_state_dict(eager.state_dict())
    opt = SGD(eager.parameters(), lr=0.02, fold_regularizers=True)
    gopt = SGD(graphed.parameters(), lr=0.02, fold_regularizers=True)

    def eager_step():
        opt.zero_grad()
        loss = model_loss(eager, ops.mse(eager(x, training=True)), True)
        opt.backward(loss)
        opt.step()
        return loss.detach()

    for _ in range(3):
        eager_step()
    step = GraphedTrainStep(graphed, lambda out, y: ops.mse(out), gopt, x, x[:1], warmup=3)
    for replay in range(4):
        le, lg = eager_step(), step()
        torch.cuda.synchronize()
        assert lg.item() == le.item(), f'replay {replay}'
        for (name, pe), (_, pg) in zip(eager.state_dict().items(), graphed.state_dict().items()):
            assert torch.equal(pg, pe), f'replay {replay}: {name}'


@pytest.mark.parametrize('kind', ['conv', 'mha', 'particle'])
def test_ebops_on_a_second_stream_change_nothing(dev, kind):
    """Inside ``ops.overlap_ebops()`` the EBOPs launches of a step (and the sum of the loss terms) run on a second stream
    when there are enough of them: same loss, same update, bit for bit, as the single-stream step."""
    from hgq2_amd import ops
    from hgq2_amd.train import SGD, model_loss
    from hgq2_amd.utils import models

    g = torch.Generator().manual_seed(33)
    if kind == 'conv':
        make = lambda: models.conv_stack(filters=8, n_out=10, device=dev)  # noqa: E731
        x, y = torch.rand(64, 12, 12, 1, generator=g).to(dev), torch.randint(0, 10, (64,), generator=g).to(dev)
        loss_fn = lambda out: ops.sparse_ce(out, y)  # noqa: E731
    elif kind == 'particle':
        make = lambda: models.particle_mlp(n_particles=8, n_features=16, hidden=(32, 16), device=dev)  # noqa: E731
        x, y = torch.randn(64, 8, 16, generator=g).to(dev), torch.randint(0, 5, (64,), generator=g).to(dev)
        loss_fn = lambda out: ops.sparse_ce(out, y)  # noqa: E731
    else:
        make = lambda: models.mha_block(num_heads=2, key_dim=8, device=dev)  # noqa: E731
        x = torch.randn(32, 12, 16, generator=g).to(dev)
        loss_fn = lambda out: ops.mse(out)  # noqa: E731
    torch.manual_seed(3)
    a = make()
    a(x, training=True)
    torch.manual_seed(3)
    b = make()
    b(x, training=True)
    b.load_state_dict(a.state_dict())
    oa, ob = SGD(a.parameters(), lr=0.02, fold_regularizers=True), SGD(b.parameters(), lr=0.02, fold_regularizers=True)
    branched = 0
    for step in range(3):
        oa.zero_grad()
        la = model_loss(a, loss_fn(a(x, training=True)), True)
        oa.backward(la)
        oa.step()
        with ops.overlap_ebops():
            ob.zero_grad()
            lb = model_loss(b, loss_fn(b(x, training=True)), True)
            branched += bool(ops._OVERLAP['pending'])
            ob.backward(lb)
            ob.step()
        assert not ops._OVERLAP['pending'] and not ops._OVERLAP['keep'], 'joined when the context is left'
        assert float(la) == float(lb), f'loss step {step}'
        for (name, pa), (_, pb) in zip(a.state_dict().items(), b.state_dict().items()):
            assert torch.equal(pa, pb), f'{name} step {step}'
    assert (branched == 3) == (kind != 'particle'), 'the attention and image models have enough EBOPs launches to branch, the per-particle one does not'


@pytest.mark.parametrize('kind', ['particle', 'conv', 'mha'])
def test_full_size_forward_matches_oracle(dev, acc64, kind):
    """The per-particle, image and attention configurations at their full sizes: one training-mode
    forward (quantized values, tracked integer bits, EBOPs) against the CPU oracle twins."""
    from hgq2_amd.utils import models

    g = torch.Generator().manual_seed(31)
    torch.manual_seed(31)
    if kind == 'particle':
        x = torch.randn(4096, 64, 16, generator=g)
        model = models.particle_mlp(device=dev)
    elif kind == 'conv':
        x = torch.rand(1024, 28, 28, 1, generator=g)
        model = models.conv_stack(device=dev)
    else:
        x = torch.randn(2048, 64, 64, generator=g)
        model = models.mha_block(device=dev)
    with torch.no_grad():
        model(x.to(dev), training=True)  # build, adapt the tracked bits
    _perturb(model, g)
    if kind == 'mha':
        r = twin.ref_mha(model, tuple(x.shape))
        with torch.no_grad():
            got = model(x.to(dev), training=True)
            want = r(x, training=True)
        _close(got, want, what='attention output')
        assert int(model._ebops.cpu().view(torch.int32)) == int(r.ebops_value)
        assert torch.equal(model._softmax.oq.quantizer._i.cpu(), r.softmax.oq.quantizer._i.detach())
        assert torch.equal(model._value_dense.iq.quantizer._i.cpu(), r.vd.iq.quantizer._i.detach())
        return
    # sequential models: walk the layers, twin each quantized one, pass the oracle's activations along
    h_p, h_r = x.to(dev), x
    with torch.no_grad():
        for layer in model.layers:
            if isinstance(layer, models.PARAMETER_FREE):
                h_p, h_r = layer(h_p), layer.host_fn(h_r)
                continue
            if kind == 'conv' and layer.__class__.__name__ == 'QConv2D':
                r = twin.ref_conv2d(layer)
            elif layer.__class__.__name__ == 'QEinsumDenseBatchnorm':
                r = twin.ref_einsum_dense_bn(layer, tuple(h_r.shape))
            else:
                r = twin.ref_dense(layer)
            h_p, h_r = layer(h_p, training=True), r(h_r, training=True)
            _close(h_p, h_r, what=f'{kind}: output of {layer.name}')
            assert torch.equal(layer.iq.quantizer._i.cpu(), r.iq.quantizer._i.detach()), layer.name
            assert int(layer.ebops.cpu().view(torch.int32)) == int(r.ebops_value), layer.name
            h_r = h_r.float()  # (float64 from the oracle's contraction; the next layer's input is fp32 on both sides)
            h_p = h_r.to(dev)  # continue from the oracle's activations so that layers are compared one by one


def test_full_size_attention_step_matches_oracle(dev):
    """QMultiHeadAttention at the full attention configuration (2048 x 64 x 64, 4 heads of 16): output,
    loss terms and the gradients of inputs, kernels and bit-widths against the oracle twin."""
    from hgq2_amd.utils import models

    g = torch.Generator().manual_seed(41)
    torch.manual_seed(41)
    x = torch.randn(2048, 64, 64, generator=g)
    layer = models.mha_block(device=dev)
    with torch.no_grad():
        layer(x.to(dev), training=True)
    _perturb(layer, g)
    r = twin.ref_mha(layer, tuple(x.shape))
    xp, xr = x.to(dev).requires_grad_(True), x.clone().requires_grad_(True)
    sm, rs = layer._softmax, r.softmax
    named_p = [('x', xp), ('wq', layer._query_dense._kernel), ('wk', layer._key_dense._kernel),
               ('wv', layer._value_dense._kernel), ('wo', layer._output_dense._kernel),
               ('q_oq_f', layer._query_dense.oq.quantizer._f), ('sm_oq_f', sm.oq.quantizer._f),
               ('v_iq_f', layer._value_dense.iq.quantizer._f), ('exp_iq_f', sm.exp_table.iq.quantizer._f),
               ('exp_oq_b', sm.exp_table.oq.quantizer._b), ('inv_iq_f', sm.inv_table.iq.quantizer._f),
               ('inv_oq_b', sm.inv_table.oq.quantizer._b)]
    named_r = [('x', xr), ('wq', r.qd.kernel), ('wk', r.kd.kernel), ('wv', r.vd.kernel), ('wo', r.od.kernel),
               ('q_oq_f', r.qd.oq.quantizer._f), ('sm_oq_f', rs.oq.quantizer._f), ('v_iq_f', r.vd.iq.quantizer._f),
               ('exp_iq_f', rs.exp_table.iq.quantizer._f), ('exp_oq_b', rs.exp_table.oq.quantizer._b),
               ('inv_iq_f', rs.inv_table.iq.quantizer._f), ('inv_oq_b', rs.inv_table.oq.quantizer._b)]
    # sums over up to 33.5 M terms: fp32 accumulation order differs between the kernels and the CPU
    _compare_step(layer, r, lambda t: layer(xp, training=t), lambda t: r(xr, training=t), named_p, named_r)
    assert int(layer._ebops.cpu().view(torch.int32)) == int(r.ebops_value)


@pytest.mark.gpu
@pytest.mark.parametrize('rows,K,N', [(1000, 16, 64), (64 * 3 + 5, 64, 32), (7, 4, 4), (70000, 64, 64), (513, 20, 12)])
def test_dense_moments_without_materialising_the_contraction(rows, K, N):
    """ops.dense_moments = (mean(z), mean(z^2)) of z = x @ w and its gradients against fp64
    (reference: the batch statistics of QEinsumDenseBatchnorm.call, einsum_dense_batchnorm.py:99-124)."""
    from hgq2_amd import ops

    dev = torch.device('cuda:0')
    g = torch.Generator().manual_seed(rows + K)
    x = torch.randn(rows, K, generator=g)
    w = torch.randn(K, N, generator=g) * 0.4
    um, us = torch.randn(N, generator=g), torch.randn(N, generator=g)
    xr, wr = x.double().requires_grad_(True), w.double().requires_grad_(True)
    z = xr @ wr
    mean_r, msq_r = z.mean(0), (z * z).mean(0)
    ((mean_r * um.double()).sum() + (msq_r * us.double()).sum()).backward()
    xd, wd = x.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
    assert ops.dense_moments_supported(xd, wd)
    mean, msq = ops.dense_moments(xd, wd)
    ((mean * um.to(dev)).sum() + (msq * us.to(dev)).sum()).backward()
    for name, got, want in (('mean', mean, mean_r), ('meansq', msq, msq_r), ('dx', xd.grad, xr.grad), ('dw', wd.grad, wr.grad)):
        scale = float(want.abs().max()) + 1e-12
        err = float((got.detach().cpu().double() - want.detach()).abs().max())
        assert err <= 1e-5 * scale, f'{name}: {err:.3e} vs scale {scale:.3e}'


@pytest.mark.gpu
@pytest.mark.parametrize('K,N,with_gamma,is_meansq', [(16, 64, True, True), (64, 32, False, True), (5, 7, True, False), (300, 130, True, True)])
def test_bn_fold_matches_the_reference_formula(K, N, with_gamma, is_meansq):
    """ops.bn_fold against get_fused_qkernel_and_qbias' algebra (einsum_dense_batchnorm.py:160-172) and
    the momentum update of call (:113-117): values against the fp32 formula, gradients against fp64 autograd."""
    from hgq2_amd import ops

    dev = torch.device('cuda:0')
    g = torch.Generator().manual_seed(K * N)
    w, bias = torch.randn(K, N, generator=g), torch.randn(N, generator=g)
    gamma = torch.rand(N, generator=g) + 0.5 if with_gamma else None
    mean = torch.randn(N, generator=g)
    spread = torch.rand(N, generator=g) + 0.1
    second = spread + mean * mean if is_meansq else spread
    mm, mv = torch.randn(N, generator=g), torch.rand(N, generator=g)
    eps, mom = 1e-7, 0.9
    up_w, up_b = torch.randn(K, N, generator=g), torch.randn(N, generator=g)
    # fp32 restatement in the reference's operation order
    var32 = second - mean * mean if is_meansq else second
    s32 = (gamma if with_gamma else 1) / torch.sqrt(var32 + eps)
    want_w, want_b = w * s32, bias + (-mean * s32)
    want_mm, want_mv = mm * mom + mean * (1.0 - mom), mv * mom + var32 * (1.0 - mom)
    # fp64 autograd for the gradients
    leaves = [t.double().requires_grad_(True) for t in (w, bias, mean, second)] + ([gamma.double().requires_grad_(True)] if with_gamma else [])
    wd, bd, md, sd = leaves[:4]
    var = sd - md * md if is_meansq else sd
    sc = (leaves[4] if with_gamma else 1.0) / torch.sqrt(var + eps)
    ((wd * sc * up_w.double()).sum() + ((bd - md * sc) * up_b.double()).sum()).backward()
    dev_leaves = [t.to(dev).requires_grad_(True) for t in (w, bias, mean, second)] + ([gamma.to(dev).requires_grad_(True)] if with_gamma else [])
    mmd, mvd = mm.to(dev), mv.to(dev)
    fw, fb = ops.bn_fold(dev_leaves[0], dev_leaves[1], dev_leaves[4] if with_gamma else None, dev_leaves[2], dev_leaves[3], is_meansq, eps,
                         mmd, mvd, mom)
    ((fw * up_w.to(dev)).sum() + (fb * up_b.to(dev)).sum()).backward()
    # sqrt and division differ by an ulp between numpy, torch-CPU and torch-GPU themselves: a few ulp here
    for name, got, want in (('fused_w', fw, want_w), ('fused_b', fb, want_b), ('moving_mean', mmd, want_mm), ('moving_var', mvd, want_mv)):
        err = float((got.detach().cpu() - want).abs().max())
        assert err <= 6e-7 * (float(want.abs().max()) + 1e-12), f'{name}: {err:.3e}'
    assert torch.equal(mmd.cpu(), want_mm)  # no sqrt / division involved
    for name, got, ref_leaf in zip(('dw', 'dbias', 'dmean', 'dsecond', 'dgamma'), dev_leaves, leaves):
        scale = float(ref_leaf.grad.abs().max()) + 1e-12
        err = float((got.grad.cpu().double() - ref_leaf.grad).abs().max())
        assert err <= 3e-5 * scale, f'{name}: {err:.3e} vs scale {scale:.3e}'


@pytest.mark.gpu
@pytest.mark.parametrize('batch,seq,heads,key_dim,oq_hom,masks', [
    (2048, 64, 4, 16, None, ''), (300, 32, 2, 8, None, ''), (37, 32, 2, 32, None, ''), (5, 64, 1, 8, None, ''),
    (70, 64, 2, 16, (0, 1), ''), (33, 32, 4, 16, (0, 1, 2), ''),
    # masks applied inside the one-pass kernels: the causal rule, a boolean mask per batch element or shared, both
    (300, 64, 4, 16, None, 'causal'), (41, 32, 2, 8, None, 'causal'), (64, 64, 2, 16, None, 'bool'), (37, 32, 2, 32, None, 'bool1'),
    (50, 64, 1, 8, (0, 1), 'causal+bool')])
def test_one_pass_attention_equals_composed_kernels(batch, seq, heads, key_dim, oq_hom, masks):
    """scores -> table softmax -> combine as one kernel each way (hgq_qattention_fwd / _bwd) against the same
    layer composing hgq_attn_scores_*, hgq_qsoftmax_* and hgq_attn_combine_*: outputs, tracked integer
    bits and loss terms bit-identical, gradients within fp32 summation noise.  With masks (reference
    src/hgq/layers/softmax.py:118-127, tests/test_mha.py:54) the composed path runs the softmax stage by stage."""
    import hgq2_amd.layers.attn.mha as mha
    from hgq2_amd.config import QuantizerConfig
    from hgq2_amd.layers import QMultiHeadAttention

    dev = torch.device('cuda:0')
    g = torch.Generator().manual_seed(batch + seq)
    torch.manual_seed(batch)
    kw = {}
    if oq_hom is not None:  # output quantizer entries shared by heads (and query positions): table rows are reused
        kw['softmax_oq_conf'] = QuantizerConfig(place='datalane', homogeneous_axis=oq_hom)
    with readme_scopes():
        layer = QMultiHeadAttention(num_heads=heads, key_dim=key_dim, **kw)
    x = torch.randn(batch, seq, heads * key_dim, generator=g)
    call_kw = {}
    if 'causal' in masks:
        call_kw['use_causal_mask'] = True
    if 'bool' in masks:
        m = torch.rand(1 if 'bool1' in masks else batch, seq, seq, generator=g) > 0.3
        m[..., 0] = True            # (every query keeps a key that the causal rule keeps, too)
        if batch > 3:
            m[min(3, m.shape[0] - 1), 5] = False     # ... except one row that is masked out altogether
        call_kw['attention_mask'] = m.to(dev)
    with torch.no_grad():
        layer(x.to(dev), training=True, **call_kw)
    _perturb(layer, g)
    state = {n: p.detach().clone() for n, p in layer.state_dict().items()}
    w = torch.randn(batch, seq, heads * key_dim, generator=g).to(dev)
    sm = layer._softmax
    params = lambda: [layer._query_dense._kernel, layer._key_dense._kernel, layer._value_dense._kernel,  # noqa: E731
                      layer._query_dense.oq.quantizer._f, layer._key_dense.oq.quantizer._f, layer._value_dense.oq.quantizer._f,
                      sm.oq.quantizer._f, sm.exp_table.iq.quantizer._f, sm.exp_table.iq.quantizer._i, sm.exp_table.oq.quantizer._b,
                      sm.exp_table.oq.quantizer._i, sm.inv_table.iq.quantizer._f, sm.inv_table.oq.quantizer._b,
                      sm.inv_table.oq.quantizer._i]
    results = []
    for fused in (True, False):
        layer.load_state_dict(state)
        mha.FUSED = fused
        try:
            xp = x.to(dev).requires_grad_(True)
            launched = []
            real = mha.ops.qattention
            mha.ops.qattention = lambda *a, **k: (launched.append(1), real(*a, **k))[1]
            try:
                y = layer(xp, training=True, **call_kw)
            finally:
                mha.ops.qattention = real
            assert bool(launched) == fused, 'the one-pass kernel runs exactly where it is switched on'
            (y * w).sum().backward()
        finally:
            mha.FUSED = True
        grads = [xp.grad.detach().clone()] + [None if p.grad is None else p.grad.detach().clone() for p in params()]
        for p in params():
            p.grad = None
        i_vars = [q.quantizer._i.detach().clone() for q in (sm.exp_table.iq, sm.inv_table.iq, sm.oq)]
        losses = [float(t.detach()) for t in layer.losses]
        mha.FUSED = fused
        try:
            with torch.no_grad():
                y_inf = layer(x.to(dev), training=False, **call_kw)  # inference mode: wrapping quantizers wrap, empty words are zeroed
        finally:
            mha.FUSED = True
        results.append((y.detach(), grads, i_vars, losses, y_inf))
    (y1, g1, i1, l1, f1), (y2, g2, i2, l2, f2) = results
    assert torch.equal(y1, y2), f'outputs differ by {float((y1 - y2).abs().max()):.3e}'
    assert torch.equal(f1, f2), f'inference outputs differ by {float((f1 - f2).abs().max()):.3e}'
    for a, b in zip(i1, i2):
        assert torch.equal(a, b)
    assert l1 == l2
    names = ['x', 'wq', 'wk', 'wv', 'q_oq_f', 'k_oq_f', 'v_oq_f', 'sm_oq_f', 'exp_iq_f', 'exp_iq_i', 'exp_oq_b', 'exp_oq_i',
             'inv_iq_f', 'inv_oq_b', 'inv_oq_i']
    for n, a, b in zip(names, g1, g2):
        assert (a is None) == (b is None), n
        if a is None:
            continue
        scale = b.abs().max().item() + 1e-12
        tol = (2e-5 if n in ('x', 'sm_oq_f') else 3e-4) * scale
        assert float((a - b).abs().max()) <= tol, f'grad {n}: {float((a - b).abs().max()):.3e} vs scale {scale:.3e}'


@pytest.mark.gpu
@pytest.mark.parametrize('oq_hom,het_table', [(None, False), ((0, 1), False), (None, True)])
def test_bit_width_algebra_ebops_kernels_match_the_layer_formulas(oq_hom, het_table):
    """hgq_lut_ebops / hgq_softmax_ebops / hgq_mha_ebops against the layers' own formulas evaluated with library
    ops (QUnaryFunctionLUT / QSoftmax / QMultiHeadAttention._compute_ebops, reference activation.py:101-104,
    softmax.py:177-206, mha.py:507-524): value and uint32 variable exactly, loss term and bit-width gradients to rounding."""
    from hgq2_amd.config import QuantizerConfig
    from hgq2_amd.layers import QMultiHeadAttention
    from hgq2_amd.quantizer.quantizer import Quantizer

    dev = torch.device('cuda:0')
    g = torch.Generator().manual_seed(17)
    kw = {}
    if oq_hom is not None:
        kw['softmax_oq_conf'] = QuantizerConfig(place='datalane', homogeneous_axis=oq_hom)
    with readme_scopes():
        layer = QMultiHeadAttention(num_heads=3, key_dim=8, parallelization_factor=5 if oq_hom else -1,
                                    softmax_allow_heterogeneous_table=het_table, **kw)
    x = torch.randn(6, 20, 24, generator=g)
    with torch.no_grad():
        layer(x.to(dev), training=True)
    _perturb(layer, g)
    sm = layer._softmax
    cases = [(layer, [(1, 20, 24)]), (sm, [(1, 3, 20, 20)]), (sm.exp_table, [(1, 3, 20, 20)]), (sm.inv_table, [(1, 3, 20, 1)])]
    fused_operand = Quantizer.bits_operand
    for obj, shapes in cases:
        params = [p for p in layer.parameters() if p.requires_grad]
        results = []
        for fused in (True, False):
            Quantizer.bits_operand = fused_operand if fused else (lambda self, shape: None)
            try:
                with torch.no_grad():
                    obj._ebops.zero_()
                term = obj._ebops_loss_term(*shapes)
                (term * 3.0).backward()
            finally:
                Quantizer.bits_operand = fused_operand
            results.append((float(term.detach()), int(obj._ebops.cpu().view(torch.int32)),
                            [None if p.grad is None else p.grad.detach().clone() for p in params]))
            for p in params:
                p.grad = None
        (t1, e1, g1), (t2, e2, g2) = results
        name = type(obj).__name__
        assert e1 == e2 and e1 > 0, (name, e1, e2)
        assert abs(t1 - t2) <= 1e-6 * abs(t2), (name, t1, t2)
        touched = 0
        for a, b in zip(g1, g2):
            assert (a is None) == (b is None) or (a is None and float(b.abs().max()) == 0.0) or (b is None and float(a.abs().max()) == 0.0), name
            if a is None or b is None:
                continue
            touched += 1
            assert float((a - b).abs().max()) <= 1e-6 * float(b.abs().max()) + 1e-12, (name, float((a - b).abs().max()))
        assert touched > 0, name


@pytest.mark.gpu
@pytest.mark.parametrize('shape,axis,center,scale', [((64, 12, 16), -1, True, True), ((32, 6, 8), 1, True, True),
                                                       ((128, 10), -1, False, True), ((40, 5, 7, 12), 3, True, False)])
def test_batch_normalization_layer(shape, axis, center, scale):
    """QBatchNormalization (reference src/hgq/layers/batch_normalization.py) against the oracle twin: output, moving
    statistics, loss terms, EBOPs and the gradients of input, gamma / beta and bit-widths."""
    from hgq2_amd.layers import QBatchNormalization

    dev = torch.device('cuda:0')
    g = torch.Generator().manual_seed(len(shape) * 10 + axis % len(shape))
    with readme_scopes():
        layer = QBatchNormalization(axis=axis, center=center, scale=scale, momentum=0.9)
    x = torch.randn(shape, generator=g) * 1.5 + 0.3
    layer(x.to(dev), training=True)
    _perturb(layer, g)
    with torch.no_grad():
        if scale:
            layer.bn_gamma.copy_(torch.rand(layer.bn_gamma.shape, generator=g) + 0.5)
        if center:
            layer.bn_beta.copy_(torch.randn(layer.bn_beta.shape, generator=g) * 0.3)
    r = twin.ref_batchnorm(layer)
    xp, xr = x.to(dev).requires_grad_(True), x.clone().requires_grad_(True)
    named_p = [('x', xp), ('iq_f', layer.iq.quantizer._f), ('kq_b', layer.kq.quantizer._b), ('kq_i', layer.kq.quantizer._i),
               ('bq_b', layer.bq.quantizer._b)]
    named_r = [('x', xr), ('iq_f', r.iq.quantizer._f), ('kq_b', r.kq.quantizer._b), ('kq_i', r.kq.quantizer._i),
               ('bq_b', r.bq.quantizer._b)]
    if scale:
        named_p.append(('gamma', layer.bn_gamma)), named_r.append(('gamma', r.gamma))
    if center:
        named_p.append(('beta', layer.bn_beta)), named_r.append(('beta', r.bn_beta))
    _compare_step(layer, r, lambda t: layer(xp, training=t), lambda t: r(xr, training=t), named_p, named_r)
    _close(layer.moving_mean, r.moving_mean, what='moving mean')
    _close(layer.moving_variance, r.moving_variance, what='moving variance')
    assert torch.equal(layer.iq.quantizer._i.cpu(), r.iq.quantizer._i.detach())
    assert int(layer.ebops.cpu().view(torch.int32)) == int(r.ebops_value)
    y_p, y_r = layer(xp, training=False), r(xr, training=False)
    _close(y_p, y_r, what='inference output')
    qs, qo = layer.qscaler_and_qoffset
    assert qs.shape == layer.moving_mean.shape and qo.shape == layer.moving_mean.shape


@pytest.mark.gpu
@pytest.mark.parametrize('rows,K,N,bw_rows', [(4096, 16, 64, 64), (640, 64, 32, 16), (70 * 64, 64, 64, 1),
                                              # narrow inputs: rows staged side by side (8, 2 and 4 of them), and the same widths where they are not
                                              (512, 8, 16, 8), (320, 32, 20, 64), (1024, 16, 8, 4), (300, 16, 8, 1), (96, 32, 64, 1), (66, 8, 4, 2)])
def test_dense_moments_with_the_input_quantizer_inside(rows, K, N, bw_rows):
    """ops.dense_moments(x, w, quant): column moments of q(x) @ w with q a training-mode WRAP quantizer applied while
    the operand is staged, against fp64 on the separately quantized input: moments, dx (straight-through), dw and the
    fractional-bit gradient sum(-ln2 (q(x) - x) dq) of this contraction."""
    from hgq2_amd import _lib, ops

    dev = torch.device('cuda:0')
    g = torch.Generator().manual_seed(rows + K + bw_rows)
    x = torch.randn(rows, K, generator=g) * 2
    w = torch.randn(K, N, generator=g) * 0.4
    f = torch.randint(2, 7, (bw_rows, K), generator=g).float()
    um, us = torch.randn(N, generator=g), torch.randn(N, generator=g)
    fr = f.repeat(rows // bw_rows, 1)
    xq = torch.floor(x * 2.0**fr + 0.5) / 2.0**fr  # RND, exact in fp32
    xr, wr = xq.double().requires_grad_(True), w.double().requires_grad_(True)
    z = xr @ wr
    mean_r, msq_r = z.mean(0), (z * z).mean(0)
    ((mean_r * um.double()).sum() + (msq_r * us.double()).sum()).backward()
    df_r = (-0.6931471805599453 * (xq.double() - x.double()) * xr.grad).view(rows // bw_rows, bw_rows, K).sum(0)
    xd, wd, fd = x.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True), f.to(dev).requires_grad_(True)
    mode = _lib.mode_bits('RND', 'WRAP', training=True, round_params=True)
    mean, msq = ops.dense_moments(xd, wd, (fd.view(-1), bw_rows, mode))
    ((mean * um.to(dev)).sum() + (msq * us.to(dev)).sum()).backward()
    for name, got, want in (('mean', mean, mean_r), ('meansq', msq, msq_r), ('dx', xd.grad, xr.grad), ('dw', wd.grad, wr.grad),
                            ('df', fd.grad, df_r)):
        want = want.detach().float()
        err = float((got.detach().cpu() - want).abs().max())
        assert err <= 1e-5 * float(want.abs().max()) + 1e-7, f'{name}: {err:.3e}'


@pytest.mark.gpu
@pytest.mark.parametrize('rows,K,N,bw_rows', [(640, 16, 64, 64), (200, 64, 32, 0), (131, 20, 12, 1), (256, 8, 32, 0), (130, 32, 16, 2), (129, 16, 16, 0)])
def test_dense_moments_chained_input_gradient(rows, K, N, bw_rows):
    """``chain=True``: the third result stands for x in a second consumer, whose gradient is added while the
    statistics' backward writes dx - equal to the unchained gradient plus that of the second consumer; the
    fractional-bit gradient of the statistics does not see it."""
    from hgq2_amd import _lib, ops

    dev = torch.device('cuda:0')
    g = torch.Generator().manual_seed(rows + K)
    x = (torch.randn(rows, K, generator=g) * 2).to(dev)
    w = (torch.randn(K, N, generator=g) * 0.4).to(dev)
    um, us, u2 = torch.randn(N, generator=g).to(dev), torch.randn(N, generator=g).to(dev), torch.randn(rows, K, generator=g).to(dev)
    quant = None
    if bw_rows:
        f = torch.randint(2, 7, (bw_rows, K), generator=g).float().to(dev)
        mode = _lib.mode_bits('RND', 'WRAP', training=True, round_params=True)
    res = []
    for chain in (False, True):
        xd, wd = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
        fd = f.clone().requires_grad_(True) if bw_rows else None
        quant = (fd.view(-1), bw_rows, mode) if bw_rows else None
        out = ops.dense_moments(xd, wd, quant, chain=chain)
        second = out[2] if chain else xd
        if chain:
            assert torch.equal(second, xd)
        ((out[0] * um).sum() + (out[1] * us).sum() + (second * second * u2).sum()).backward()
        res.append((out[0].detach(), out[1].detach(), xd.grad, wd.grad, fd.grad if bw_rows else None))
    for name, a, b in zip(('mean', 'meansq', 'dx', 'dw', 'df'), *res):
        if a is None:
            continue
        if name == 'dx':  # the sum is formed in a different order
            assert float((a - b).abs().max()) <= 1e-6 * float(a.abs().max()), name
        else:
            assert torch.equal(a, b), name


@pytest.mark.gpu
@pytest.mark.parametrize('shape', [(4096, 64, 32), (3, 1, 5), (17, 100, 7), (2, 300, 1028), (5, 9, 260), (0, 4, 8)])
def test_mean_over_the_middle_axis(shape):
    """ops.mean_mid == x.mean(1) and its gradient (fp64 reference), the form the global average pooling layers and the
    mean over the particles take on the GPU."""
    from hgq2_amd import ops

    dev = torch.device('cuda:0')
    g = torch.Generator().manual_seed(sum(shape))
    x = torch.randn(shape, generator=g)
    up = torch.randn(shape[0], shape[2], generator=g)
    xd = x.to(dev).requires_grad_(True)
    y = ops.mean_mid(xd)
    assert tuple(y.shape) == (shape[0], shape[2])
    if shape[0] == 0:
        return
    want = x.double().mean(1)
    assert float((y.detach().cpu().double() - want).abs().max()) <= 1e-6 * (float(want.abs().max()) + 1e-6)
    (y * up.to(dev)).sum().backward()
    want_dx = (up.double() / shape[1]).unsqueeze(1).expand(shape)
    assert float((xd.grad.cpu().double() - want_dx).abs().max()) <= 1e-6 * float(want_dx.abs().max())


@pytest.mark.gpu
@pytest.mark.parametrize('groups,mean_rows,K,N,bw_rows,act,bias', [(4096, 64, 64, 32, 64, 'relu', True), (37, 64, 16, 64, 1, 'relu', True),
                                                               (9, 32, 32, 20, 32, 'none', True), (130, 32, 8, 4, 0, 'relu', False),
                                                               (1, 64, 48, 64, 2, 'relu', True), (3, 32, 64, 64, 16, 'none', False)])
def test_contraction_with_the_mean_over_row_groups(groups, mean_rows, K, N, bw_rows, act, bias):
    """ops.qdense_mean (the contraction kernel writes the means of groups of 32 / 64 output rows; its backward reads the
    means' gradient with a zero row stride) against ops.qdense followed by ops.mean_mid: same means, and the same gradients
    of the input, the kernel, the bias and the fractional bits, to the accumulation order of fp32 sums."""
    from hgq2_amd import _lib, ops

    dev = torch.device('cuda:0')
    rows = groups * mean_rows
    g = torch.Generator().manual_seed(groups + K + N)
    x = (torch.randn(rows, K, generator=g) * 2).to(dev)
    w = (torch.randint(-32, 32, (K, N), generator=g).float() / 16).to(dev)
    b = (torch.randint(-8, 8, (N,), generator=g).float() / 8).to(dev) if bias else None
    up = torch.randn(groups, N, generator=g).to(dev)
    act_code = _lib.ACT_RELU if act == 'relu' else _lib.ACT_NONE
    mode = _lib.mode_bits('RND', 'WRAP', training=True, round_params=True) if bw_rows else 0
    if bw_rows:
        f = torch.randint(2, 7, (bw_rows, K), generator=g).float().to(dev)
        k = torch.ones(bw_rows * K, dtype=torch.uint8, device=dev)
        i = torch.full((bw_rows * K,), 4.0, device=dev)
    if not _lib.load().hgq_dense_use_bf16_parts(-1):
        assert not ops.qdense_mean_supported(rows, K, N, bw_rows, mean_rows, mode)
        pytest.skip('the fused mean rides on the bf16-part kernels')
    assert ops.qdense_mean_supported(rows, K, N, bw_rows, mean_rows, mode)
    res = []
    for fused in (False, True):
        xd, wd = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
        bd = b.clone().requires_grad_(True) if bias else None
        fd = f.clone().requires_grad_(True) if bw_rows else None
        if fused:
            m, amax = ops.qdense_mean(xd, k if bw_rows else None, fd.view(-1) if bw_rows else None, wd, bd, act_code, mode, bw_rows, mean_rows)
        else:
            y, amax = ops.qdense(xd, k if bw_rows else None, i if bw_rows else None, fd.view(-1) if bw_rows else None, wd, bd, act_code, mode,
                                 bw_rows, bool(bw_rows))
            m = ops.mean_mid(y.view(groups, mean_rows, N))
        (m * up).sum().backward()
        res.append((m.detach(), amax, xd.grad, wd.grad, bd.grad if bias else None, fd.grad if bw_rows else None))
    assert tuple(res[1][0].shape) == (groups, N)
    assert torch.equal(res[0][1], res[1][1]), 'abs-max slices of the input quantizer'
    for name, a, c in zip(('means', 'amax', 'dx', 'dw', 'db', 'df'), *res):
        if a is None or name == 'amax':
            continue
        err = float((a.double() - c.double()).abs().max())
        assert err <= 2e-6 * float(a.abs().max()) + 1e-9, f'{name}: {err:.3e} of {float(a.abs().max()):.3e}'


@pytest.mark.gpu
@pytest.mark.parametrize('with_batchnorm', [True, False])
def test_a_contraction_layer_takes_the_mean_over_the_positions_with_it(dev, with_batchnorm, monkeypatch):
    """``Sequential([QEinsumDense(Batchnorm)('bpf,fh->bph', relu), GlobalAveragePooling1D, ...])``: the pair runs as one
    operator each way (``ops.qdense_mean``); two training steps give the outputs, losses, gradients and states of the same
    model run layer by layer."""
    from hgq2_amd import _lib, host, ops
    from hgq2_amd.core import Sequential
    from hgq2_amd.layers import QDense, QEinsumDense, QEinsumDenseBatchnorm
    from hgq2_amd.train import SGD, model_loss

    calls = []
    real = ops.qdense_mean
    monkeypatch.setattr(ops, 'qdense_mean', lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    g = torch.Generator().manual_seed(3)
    x = torch.randn(48, 64, 16, generator=g).to(dev)
    models = []
    for absorb in (True, False):
        torch.manual_seed(11)
        with readme_scopes():
            cls = QEinsumDenseBatchnorm if with_batchnorm else QEinsumDense
            first = cls('bpf,fh->bph', (64, 32), bias_axes='h', activation='relu')
            model = Sequential([first, host.GlobalAveragePooling1D(), QDense(5)])
        model(x, training=False)
        _perturb(model, torch.Generator().manual_seed(5))
        if not absorb:
            first.absorbs = lambda nxt, xx: False
        models.append(model)
    outs = []
    for model in models:
        opt = SGD(model.parameters(), lr=0.01)
        hist = []
        for t in range(2):
            opt.zero_grad()
            out = model(x, training=True)
            loss = model_loss(model, (out * out).mean())
            if t == 0:
                loss.backward()  # every gradient through autograd: the operator's backward with its own slice reduction
            else:
                opt.backward(loss)  # gradient sink open: slices left for the joint reduction, pieces parked on the variables
            grads = {n: p.grad.clone() for n, p in model.named_parameters() if p.grad is not None}
            opt.step()
            hist.append((out.detach().clone(), loss.detach().clone(), grads))
        outs.append((hist, {n: v.detach().clone() for n, v in model.state_dict().items()}))
    # once per training step of the absorbing model only (never on the fp32 matrix instruction: the pair then runs in two steps)
    assert len(calls) == (2 if _lib.load().hgq_dense_use_bf16_parts(-1) else 0)
    (ha, sa), (hb, sb) = outs
    for (oa, la, ga), (ob, lb, gb) in zip(ha, hb):
        _close(oa, ob.cpu(), what='output')
        _close(la, lb.cpu(), what='loss')
        assert ga.keys() == gb.keys()
        for n in ga:
            _close(ga[n], gb[n].cpu(), rtol=2e-5, what=f'grad {n}')
    assert sa.keys() == sb.keys()
    for n in sa:
        _close(sa[n].float(), sb[n].float().cpu(), rtol=2e-5, what=f'state {n}')


@pytest.mark.gpu
def test_global_average_pooling_layers_use_it_and_match_the_library_mean():
    from hgq2_amd.config import QuantizerConfigScope
    from hgq2_amd.layers import QGlobalAveragePooling1D, QGlobalAveragePooling2D

    dev = torch.device('cuda:0')
    g = torch.Generator().manual_seed(8)
    with QuantizerConfigScope(default_q_type='dummy'):
        for layer, shape in ((QGlobalAveragePooling1D(enable_ebops=False), (6, 10, 12)),
                             (QGlobalAveragePooling2D(enable_ebops=False, keepdims=True), (3, 5, 7, 8))):
            x = torch.randn(shape, generator=g)
            y = layer(x.to(dev), training=False)
            want = x.mean(dim=tuple(range(1, len(shape) - 1)), keepdim=layer.keepdims)
            assert y.shape == want.shape
            assert torch.allclose(y.cpu(), want, rtol=1e-6, atol=1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize('factor,het', [(-1, True), (3, True), (7, False)])
def test_pooling_ebops_in_one_launch(dev, factor, het, monkeypatch):
    """The pooling layers' EBOPs (reference src/hgq/layers/pooling.py:28-30: sum(bits) * parallelization_factor / n_parallel)
    through ``hgq_sum_ebops``: the uint32 variable, the loss term and the bit-width gradients equal those of the formula
    written in tensor operations, also where the factor does not divide."""
    from hgq2_amd import ops
    from hgq2_amd.layers import QAveragePooling2D
    from hgq2_amd.layers.core.base import QLayerBase
    from hgq2_amd.train import model_loss

    kinds = []
    real = ops.bits_ebops
    monkeypatch.setattr(ops, 'bits_ebops', lambda kind, *a, **k: (kinds.append(kind), real(kind, *a, **k))[1])
    g = torch.Generator().manual_seed(5)
    x = torch.randn(6, 8, 10, 4, generator=g).to(dev)
    res = []
    for fused in (True, False):
        torch.manual_seed(2)
        with readme_scopes(beta0=1e-3):
            layer = QAveragePooling2D((2, 2), parallelization_factor=factor)
        layer(x, training=False)
        if het:
            _perturb(layer, torch.Generator().manual_seed(9))
        if not fused:  # the same layer on the base class's formula
            layer._ebops_loss_term = lambda shape, layer=layer: QLayerBase._ebops_loss_term(layer, shape)
        out = layer(x, training=True)
        loss = model_loss(layer, (out * out).mean())
        loss.backward()
        q = layer.iq.quantizer
        res.append((int(layer._ebops.view(torch.int32)), loss.detach(), q._f.grad.clone(), q._i.grad.clone() if q._i.grad is not None else None))
    assert kinds == ['sum']
    (ea, la, fa, ia), (eb, lb, fb, ib) = res
    assert ea == eb and ea > 0
    _close(la, lb.cpu(), what='loss')
    _close(fa, fb.cpu(), what='d/df')
    if ia is not None:
        _close(ia, ib.cpu(), what='d/di')


@pytest.mark.parametrize('kind', ['conv', 'particle'])
def test_plain_backward_inside_the_overlap_context(dev, kind):
    """``model_loss`` inside ``ops.overlap_ebops()`` returns a total whose value is written later; ``loss.backward()`` -
    without the optimizer's gradient sink - still gives the gradients of the step outside the context, and the value is
    there when the context is left."""
    from hgq2_amd import ops
    from hgq2_amd.train import SGD, model_loss
    from hgq2_amd.utils import models

    g = torch.Generator().manual_seed(34)
    if kind == 'conv':
        make = lambda: models.conv_stack(filters=8, n_out=10, device=dev)  # noqa: E731
        x, y = torch.rand(64, 12, 12, 1, generator=g).to(dev), torch.randint(0, 10, (64,), generator=g).to(dev)
    else:
        make = lambda: models.particle_mlp(n_particles=8, n_features=16, hidden=(32, 16), device=dev)  # noqa: E731
        x, y = torch.randn(64, 8, 16, generator=g).to(dev), torch.randint(0, 5, (64,), generator=g).to(dev)
    torch.manual_seed(4)
    a = make()
    a(x, training=True)
    torch.manual_seed(4)
    b = make()
    b(x, training=True)
    b.load_state_dict(a.state_dict())
    oa, ob = SGD(a.parameters(), lr=0.02), SGD(b.parameters(), lr=0.02)
    for step in range(2):
        oa.zero_grad()
        la = model_loss(a, ops.sparse_ce(a(x, training=True), y))
        la.backward()
        oa.step()
        with ops.overlap_ebops():
            ob.zero_grad()
            lb = model_loss(b, ops.sparse_ce(b(x, training=True), y))
            assert lb.requires_grad
            lb.backward()
            ob.step()
        assert float(la) == float(lb), f'loss step {step}'
        for (name, pa), (_, pb) in zip(a.state_dict().items(), b.state_dict().items()):
            assert torch.equal(pa, pb), f'{name} step {step}'
