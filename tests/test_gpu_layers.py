"""GPU parity of the layer API (hgq2_amd.layers / quantizer / config) against the CPU oracle's
restatement of the reference's Python, on identical weights and inputs."""

import math

import numpy as np
import pytest
import torch

from oracle import hgq_ref as ref

pytestmark = pytest.mark.gpu
RTOL = 1e-5


def _copy_mlp(src: 'ref.RefMLP', model, dev):
    """Load the oracle's weights and bit-widths into the product model."""
    with torch.no_grad():
        for rl, pl in zip(src.layers, model.layers):
            pl._kernel.copy_(rl.kernel.detach().to(dev))
            pl.bias.copy_(rl.bias.detach().to(dev))
            for rq, pq in ((rl.iq, pl.iq), (rl.kq, pl.kq), (rl.bq, pl.bq)):
                for name, t in rq.quantizer.variables().items():
                    getattr(pq.quantizer, name).copy_(t.detach().to(dev))


def _close(got, want, scale=None, rtol=RTOL, what=''):
    got, want = got.detach().double().cpu(), want.detach().double()
    tol = rtol * (want.abs() if scale is None else scale) + 1e-12
    err = (got - want).abs()
    assert torch.all(err <= tol), f'{what}: max err {err.max():.3e}, tol {tol.max():.3e}'


def test_scopes_produce_reference_default_configs():
    from hgq2_amd.utils.models import qdense_mlp
    from hgq2_amd.quantizer.internal import FixedPointQuantizerKBI, FixedPointQuantizerKIF

    m = qdense_mlp(device='cpu')
    l0 = m.layers[0]
    assert isinstance(l0.iq.quantizer, FixedPointQuantizerKIF) and l0.iq.quantizer.overflow_mode == 'WRAP'
    assert isinstance(l0.kq.quantizer, FixedPointQuantizerKBI) and l0.kq.quantizer.overflow_mode == 'SAT_SYM'
    assert isinstance(l0.bq.quantizer, FixedPointQuantizerKBI) and l0.bq.quantizer.overflow_mode == 'SAT_SYM'
    assert tuple(l0.iq.quantizer._i.shape) == (1, 16) and tuple(l0.kq.quantizer._b.shape) == (16, 64)
    assert l0.iq.quantizer._k.dtype == torch.uint8 and l0._ebops.dtype == torch.uint32


@pytest.mark.parametrize('batch', (16384, 1000))
def test_mlp_training_steps_match_oracle(dev, acc64, batch):
    from hgq2_amd import ops
    from hgq2_amd.train import SGD, model_loss
    from hgq2_amd.utils.models import qdense_mlp

    g = torch.Generator().manual_seed(0)
    x = torch.randn(batch, 16, generator=g)
    labels = torch.randint(0, 5, (batch,), generator=g)
    oracle = ref.RefMLP(seed=1)
    model = qdense_mlp(device=dev)
    _copy_mlp(oracle, model, dev)
    opt = SGD(model.parameters(), lr=0.01)
    xd, yd = x.to(dev), labels.to(dev)
    for step in range(3):
        want_loss, want_logits = oracle.train_step(x, labels, lr=0.01)
        opt.zero_grad()
        logits = model(xd, training=True)
        loss = model_loss(model, ops.sparse_ce(logits, yd))
        loss.backward()
        opt.step()
        _close(logits, want_logits, scale=want_logits.abs() + 1.0, rtol=1e-5, what=f'logits step {step}')
        assert abs(loss.item() - want_loss.item()) <= 1e-5 * abs(want_loss.item())
        for n, (rl, pl) in enumerate(zip(oracle.layers, model.layers)):
            # tracked integer bits and EBOPs: exact
            assert torch.equal(pl.iq.quantizer._i.cpu(), rl.iq.quantizer._i.detach()), f'layer {n} _i step {step}'
            assert int(pl.ebops.cpu().view(torch.int32)) == int(rl.ebops_value), f'layer {n} ebops step {step}'
            _close(pl._kernel, rl.kernel, scale=rl.kernel.detach().abs() + 1e-3, what=f'kernel {n}')
            _close(pl.bias, rl.bias, scale=rl.bias.detach().abs() + 1e-3, what=f'bias {n}')
            _close(pl.iq.quantizer._f, rl.iq.quantizer._f, scale=rl.iq.quantizer._f.detach().abs() + 1e-3, what=f'iq._f {n}')
            _close(pl.kq.quantizer._b, rl.kq.quantizer._b, scale=rl.kq.quantizer._b.detach().abs() + 1e-3, what=f'kq._b {n}')
            _close(pl.kq.quantizer._i, rl.kq.quantizer._i, scale=rl.kq.quantizer._i.detach().abs() + 1e-3, what=f'kq._i {n}')
            _close(pl.bq.quantizer._b, rl.bq.quantizer._b, scale=rl.bq.quantizer._b.detach().abs() + 1e-3, what=f'bq._b {n}')


def test_mlp_inference_matches_oracle_bitexact_inputs(dev, acc64):
    """Inference mode (WRAP applied, empty words zeroed): quantized activations are exact; the
    logits are compared at 1e-5."""
    from hgq2_amd.utils.models import qdense_mlp

    g = torch.Generator().manual_seed(3)
    x = torch.randn(4096, 16, generator=g) * 3
    oracle = ref.RefMLP(seed=2)
    model = qdense_mlp(device=dev)
    with torch.no_grad():
        for layer in oracle.layers:  # make the first layer overflow and one lane empty
            layer.iq.quantizer._i.fill_(1.0)
        oracle.layers[0].iq.quantizer._f[0, 3] = -2.0
        oracle.layers[0].iq.quantizer._k[0, 3] = 0
    _copy_mlp(oracle, model, dev)
    with torch.no_grad():
        want = oracle.forward(x, training=False)
        got = model(x.to(dev), training=False)
        q0 = model.layers[0].iq(x.to(dev), training=False)
        w0 = oracle.layers[0].iq(x, training=False)
    assert torch.equal(q0.cpu(), w0)
    assert torch.all(q0[:, 3] == 0)
    _close(got, want, scale=want.abs() + 1.0, rtol=1e-5, what='logits')


def test_graphed_step_equals_eager_steps(dev):
    """HIP-graph replays of the training step give the same trajectory as eager steps."""
    from hgq2_amd import ops
    from hgq2_amd.train import SGD, GraphedTrainStep, model_loss
    from hgq2_amd.utils.models import qdense_mlp

    g = torch.Generator().manual_seed(5)
    xs = [torch.randn(2048, 16, generator=g).to(dev) for _ in range(4)]
    ys = [torch.randint(0, 5, (2048,), generator=g).to(dev) for _ in range(4)]
    src = ref.RefMLP(seed=4)

    eager = qdense_mlp(device=dev)
    _copy_mlp(src, eager, dev)
    opt = SGD(eager.parameters(), lr=0.01, fold_regularizers=True)
    graphed = qdense_mlp(device=dev)
    _copy_mlp(src, graphed, dev)
    gopt = SGD(graphed.parameters(), lr=0.01, fold_regularizers=True)
    # capture warms up on (and therefore trains on) its example batch: give both models the same history
    warm = 3
    def eager_step(x, y):
        # the step as the captured one runs it: EBOPs launches on the second stream, gradient pieces through the sink
        opt.zero_grad()
        with ops.overlap_ebops():
            loss = model_loss(eager, ops.sparse_ce(eager(x, training=True), y), True)
            opt.backward(loss)
            opt.step()
        return loss

    for _ in range(warm + 1):
        eager_step(xs[0], ys[0])
    step = GraphedTrainStep(graphed, ops.sparse_ce, gopt, xs[0], ys[0], warmup=warm)
    step()  # first replay = the (warm+1)-th step on the example batch
    for x, y in zip(xs[1:], ys[1:]):
        loss = eager_step(x, y)
        gl = step(x, y)
        torch.cuda.synchronize()
        # the same launches in the same order on the same numbers: bit for bit
        assert gl.item() == loss.item()
        for pe, pg in zip(eager.parameters(), graphed.parameters()):
            assert torch.equal(pg, pe)
        for le, lg in zip(eager.layers, graphed.layers):
            assert torch.equal(le.iq.quantizer._i, lg.iq.quantizer._i)
            assert int(le.ebops.cpu().view(torch.int32)) == int(lg.ebops.cpu().view(torch.int32))


@pytest.mark.parametrize('batch,dims', [(16384, (16, 64, 32, 32, 5)), (1000, (16, 64, 32, 32, 5)), (300, (7, 40, 3))])
def test_fused_qdense_stack_step_matches_oracle(dev, acc64, batch, dims):
    """The whole-step kernels update every variable as the oracle's layer-by-layer step does."""
    from hgq2_amd.train import FusedQDenseStack
    from hgq2_amd.utils.models import qdense_mlp

    g = torch.Generator().manual_seed(7)
    x = torch.randn(batch, dims[0], generator=g)
    labels = torch.randint(0, dims[-1], (batch,), generator=g)
    oracle = ref.RefMLP(dims=dims, seed=3)
    model = qdense_mlp(dims, device=dev)
    _copy_mlp(oracle, model, dev)
    fused = FusedQDenseStack(model, lr=0.01)
    xd, yd = x.to(dev), labels.to(dev)
    for step in range(3):
        want_loss, _ = oracle.train_step(x, labels, lr=0.01)
        loss = fused.step(xd, yd)
        assert abs(loss.item() - want_loss.item()) <= 1e-5 * abs(want_loss.item()), f'loss step {step}'
        for n, (rl, pl) in enumerate(zip(oracle.layers, model.layers)):
            assert torch.equal(pl.iq.quantizer._i.cpu(), rl.iq.quantizer._i.detach()), f'layer {n} _i step {step}'
            assert int(pl.ebops.cpu().view(torch.int32)) == int(rl.ebops_value), f'layer {n} ebops step {step}'
            _close(pl._kernel, rl.kernel, scale=rl.kernel.detach().abs() + 1e-3, what=f'kernel {n}')
            _close(pl.bias, rl.bias, scale=rl.bias.detach().abs() + 1e-3, what=f'bias {n}')
            _close(pl.iq.quantizer._f, rl.iq.quantizer._f, scale=rl.iq.quantizer._f.detach().abs() + 1e-3, what=f'iq._f {n}')
            _close(pl.kq.quantizer._b, rl.kq.quantizer._b, scale=rl.kq.quantizer._b.detach().abs() + 1e-3, what=f'kq._b {n}')
            _close(pl.kq.quantizer._i, rl.kq.quantizer._i, scale=rl.kq.quantizer._i.detach().abs() + 1e-3, what=f'kq._i {n}')
            _close(pl.bq.quantizer._b, rl.bq.quantizer._b, scale=rl.bq.quantizer._b.detach().abs() + 1e-3, what=f'bq._b {n}')
            _close(pl.bq.quantizer._i, rl.bq.quantizer._i, scale=rl.bq.quantizer._i.detach().abs() + 1e-3, what=f'bq._i {n}')


def test_gradient_pieces_of_variables_the_optimizer_does_not_own_go_through_autograd(dev):
    """``SGD.backward`` parks EBOPs gradient pieces on the variables for its own update kernel.  A variable that this
    optimizer does not step (here: every bit-width variable) must get its whole gradient in ``.grad`` instead - the same
    values a plain ``loss.backward()`` gives."""
    from hgq2_amd import ops
    from hgq2_amd.train import SGD, model_loss
    from hgq2_amd.utils.models import qdense_mlp

    g = torch.Generator().manual_seed(12)
    x = torch.randn(512, 16, generator=g).to(dev)
    y = torch.randint(0, 5, (512,), generator=g).to(dev)
    model = qdense_mlp(device=dev)
    _copy_mlp(ref.RefMLP(seed=6), model, dev)
    model(x, training=True)
    named = dict(model.named_parameters())
    weights = [p for n, p in named.items() if n.endswith('_kernel') or n.endswith('bias')]
    others = {n: p for n, p in named.items() if p.requires_grad and all(p is not w for w in weights)}
    assert weights and others
    state = {n: t.detach().clone() for n, t in model.state_dict().items()}

    def grads(sink):
        model.load_state_dict(state)
        for p in named.values():
            p.grad = None
            p._hgq_side = None
        loss = model_loss(model, ops.sparse_ce(model(x, training=True), y))
        if sink:
            SGD(weights, lr=0.01).backward(loss)
        else:
            loss.backward()
        return {n: p.grad.detach().clone() for n, p in others.items()}

    plain, with_sink = grads(False), grads(True)
    for n in others:
        assert not getattr(others[n], '_hgq_side', None), f'{n}: a piece was parked where no optimizer reads it'
        assert torch.equal(plain[n], with_sink[n]), n


def test_fused_qdense_stack_step_is_the_same_bits_on_every_run(dev):
    """131 072 rows = eight tiles per workgroup: a workgroup's gradient sums run over several tiles and the loss is put
    together from the pieces of ~80 workgroups.  No floating-point sum of the two launches depends on the order in which
    wavefronts or workgroups arrive, so two runs from the same state leave the same bits in every variable and in the loss."""
    from hgq2_amd.train import FusedQDenseStack
    from hgq2_amd.utils.models import qdense_mlp

    dims = (16, 64, 32, 32, 5)
    g = torch.Generator().manual_seed(9)
    x = torch.randn(131072, dims[0], generator=g).to(dev)
    labels = torch.randint(0, dims[-1], (131072,), generator=g).to(dev)
    src = ref.RefMLP(dims=dims, seed=5)
    runs = []
    for _ in range(2):
        model = qdense_mlp(dims, device=dev)
        _copy_mlp(src, model, dev)
        fused = FusedQDenseStack(model, lr=0.01)
        losses = [fused.step(x, labels).clone() for _ in range(3)]
        torch.cuda.synchronize()
        runs.append((losses, {n: p.detach().clone() for n, p in model.state_dict().items()}))
    (l1, s1), (l2, s2) = runs
    for a, b in zip(l1, l2):
        assert torch.equal(a, b), f'loss {a.item()!r} vs {b.item()!r}'
    assert s1.keys() == s2.keys()
    for n in s1:
        assert torch.equal(s1[n], s2[n]), n


def test_fused_step_reports_a_label_outside_the_classes_and_recovers(dev):
    """A label outside [0, classes) makes the step's loss NaN (the piece travels beside the fixed-point sum of the loss
    pieces) and contributes no cross-entropy gradient; the next step with valid labels reports a finite loss again, the
    one a stack that never saw the bad batch reports from the same variables."""
    from hgq2_amd.train import FusedQDenseStack
    from hgq2_amd.utils.models import qdense_mlp

    dims = (16, 64, 32, 32, 5)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(4096, dims[0], generator=g).to(dev)
    labels = torch.randint(0, dims[-1], (4096,), generator=g).to(dev)
    bad = labels.clone()
    bad[17] = dims[-1]
    bad[4000] = -1
    src = ref.RefMLP(dims=dims, seed=6)
    model = qdense_mlp(dims, device=dev)
    _copy_mlp(src, model, dev)
    fused = FusedQDenseStack(model, lr=0.01)
    assert math.isfinite(float(fused.step(x, labels)))
    assert math.isnan(float(fused.step(x, bad)))
    state = {n: p.detach().clone() for n, p in model.state_dict().items()}
    assert all(bool(torch.isfinite(v.float()).all()) for v in state.values()), 'the bad labels reached a variable'
    after = float(fused.step(x, labels))
    assert math.isfinite(after)
    twin = qdense_mlp(dims, device=dev)
    twin.load_state_dict(state)
    assert float(FusedQDenseStack(twin, lr=0.01).step(x, labels)) == after


def test_fused_stack_with_an_activation_on_the_output_layer(dev, acc64):
    """QDense applies its activation whatever follows it (reference src/hgq/layers/core/dense.py:66-67): with relu on the
    last layer the cross-entropy gradient passes the relu mask before it reaches that layer's kernel."""
    import torch.nn.functional as F

    from hgq2_amd.config import LayerConfigScope, QuantizerConfigScope
    from hgq2_amd.core import Sequential
    from hgq2_amd.layers import QDense
    from hgq2_amd.train import FusedQDenseStack
    from oracle import twin

    g = torch.Generator().manual_seed(11)
    torch.manual_seed(11)
    x = torch.randn(500, 9, generator=g)
    labels = torch.randint(0, 6, (500,), generator=g)
    with QuantizerConfigScope(place='all', default_q_type='kbi', overflow_mode='SAT_SYM'), \
            QuantizerConfigScope(place='datalane', default_q_type='kif', overflow_mode='WRAP'), \
            LayerConfigScope(enable_ebops=True, beta0=1e-5):
        layers = [QDense(20, activation='relu'), QDense(6, activation='relu')]
    model = Sequential(layers)
    xd, yd = x.to(dev), labels.to(dev)
    model(xd, training=True)
    refs = [twin.ref_dense(layer) for layer in layers]
    fused = FusedQDenseStack(model, lr=0.05)
    for step in range(3):
        variables = [v for r in refs for v in r.trainable_variables()]
        for v in variables:
            v.grad = None
        h = x
        for r in refs:
            h = r(h, training=True)
        assert bool((h == 0).any()), 'the case needs clipped outputs'
        want_loss = F.cross_entropy(h.float(), labels)
        for r in refs:
            want_loss = want_loss + r.extra_loss()
        want_loss.backward()
        with torch.no_grad():
            for v in variables:
                if v.grad is not None:
                    v.sub_(0.05 * v.grad)
        for r in refs:
            r.apply_constraints()
        loss = fused.step(xd, yd)
        assert abs(loss.item() - want_loss.item()) <= 1e-5 * abs(want_loss.item()), f'loss step {step}'
        for n, (rl, pl) in enumerate(zip(refs, layers)):
            assert torch.equal(pl.iq.quantizer._i.cpu(), rl.iq.quantizer._i.detach()), f'layer {n} _i step {step}'
            assert int(pl.ebops.cpu().view(torch.int32)) == int(rl.ebops_value), f'layer {n} ebops step {step}'
            _close(pl._kernel, rl.kernel, scale=rl.kernel.detach().abs() + 1e-3, what=f'kernel {n} step {step}')
            _close(pl.bias, rl.bias, scale=rl.bias.detach().abs() + 1e-3, what=f'bias {n} step {step}')
            _close(pl.iq.quantizer._f, rl.iq.quantizer._f, scale=rl.iq.quantizer._f.detach().abs() + 1e-3, what=f'iq._f {n}')
            _close(pl.kq.quantizer._b, rl.kq.quantizer._b, scale=rl.kq.quantizer._b.detach().abs() + 1e-3, what=f'kq._b {n}')


def test_fused_step_reuses_its_weight_image_only_while_it_owns_the_variables(dev):
    """Steps that reuse the quantized weight image left by the previous update are bit-identical to
    steps that quantize the variables again, across a change of batch size, and an in-place change
    of a variable from outside (seen through the tensor's version counter) is picked up."""
    from hgq2_amd.train import FusedQDenseStack
    from hgq2_amd.utils.models import qdense_mlp

    g = torch.Generator().manual_seed(11)
    xs = [torch.randn(n, 16, generator=g).to(dev) for n in (700, 700, 256, 700, 700)]
    ys = [torch.randint(0, 5, (x.shape[0],), generator=g).to(dev) for x in xs]
    oracle = ref.RefMLP(seed=5)
    models = [qdense_mlp(device=dev) for _ in range(2)]
    for m in models:
        _copy_mlp(oracle, m, dev)
    cached, fresh = (FusedQDenseStack(m, lr=0.05) for m in models)
    for step, (x, y) in enumerate(zip(xs, ys)):
        if step == 3:  # an outside change of a kernel entry, on both models
            for m in models:
                with torch.no_grad():
                    m.layers[1]._kernel[3, 4] += 0.25
        fresh._versions = None  # always quantize again
        la, lb = cached.step(x, y), fresh.step(x, y)
        # the reported loss is the sum of some eighty terms (cross-entropy, EBOPs and regularisation terms of every update
        # workgroup) added with atomics: equal up to the order of those fp32 adds
        assert abs(float(la) - float(lb)) <= 5e-6 * abs(float(lb)), f'loss step {step}'
        for pa, pb in zip(models[0].parameters(), models[1].parameters()):
            assert torch.equal(pa, pb), f'step {step}'


def test_trace_minmax_matches_oracle(dev, acc64):
    """The calibration pass (training='tracing') leaves the same integer bits, keep-negative flags
    and EBOPs as the oracle, and inference after it is bit-identical."""
    from hgq2_amd.utils import trace_minmax
    from hgq2_amd.utils.models import qdense_mlp

    g = torch.Generator().manual_seed(8)
    data = torch.randn(3000, 16, generator=g) * 1.5
    oracle = ref.RefMLP(seed=2)
    model = qdense_mlp(device=dev)
    _copy_mlp(oracle, model, dev)
    total = trace_minmax(model, data.numpy(), batch_size=1024)
    for rl in oracle.layers:  # reset, then three calibration batches
        q = rl.iq.quantizer
        with torch.no_grad():
            q._i.fill_(-1e9)
            q._k.zero_()
    from hgq2_amd.core import TrainingFlagWrapper

    for s in range(0, 3000, 1024):  # the flag object is falsy and compares equal to 'tracing', as in the reference
        oracle.forward(data[s:s + 1024], training=TrainingFlagWrapper('tracing'))
    for rl, pl in zip(oracle.layers, model.layers):
        assert torch.equal(pl.iq.quantizer._i.cpu(), rl.iq.quantizer._i.detach())
        assert torch.equal(pl.iq.quantizer._k.cpu(), rl.iq.quantizer._k)
        assert int(pl.ebops.cpu().view(torch.int32)) == int(rl.ebops_value)
    assert total == sum(int(rl.ebops_value) for rl in oracle.layers)
    with torch.no_grad():
        got = model(data[:512].to(dev), training=False)
        want = oracle.forward(data[:512], training=False)
    _close(got, want, scale=want.abs() + 1.0, rtol=1e-5, what='logits after calibration')
    # continuing without a reset only ever widens
    before = [pl.iq.quantizer._i.clone() for pl in model.layers]
    out = trace_minmax(model, (data[:100] * 4).numpy(), reset=False, return_results=True)
    assert out.shape == (100, 5)
    for b, pl in zip(before, model.layers):
        assert torch.all(pl.iq.quantizer._i >= b)


@pytest.mark.gpu
@pytest.mark.parametrize('n,with_target', [(1, False), (7, True), (4096 * 33 + 3, True), (2048 * 64 * 64, False)])
def test_mse_loss_and_gradient(n, with_target):
    """ops.mse against the fp64 definition mean((pred - target)^2) and its gradient 2 (pred - target) / n
    scaled by the upstream gradient; run twice: the fixed summation order gives the same bits."""
    from hgq2_amd import ops

    dev = torch.device('cuda:0')
    g = torch.Generator().manual_seed(n % 1000)
    pred = torch.randn(n, generator=g)
    target = torch.randn(n, generator=g) if with_target else None
    ref_d = pred.double() - (target.double() if with_target else 0.0)
    want = float((ref_d * ref_d).mean())
    p = pred.to(dev).requires_grad_(True)
    t = target.to(dev) if with_target else None
    loss = ops.mse(p, t)
    (loss * 3.0).backward()
    assert abs(float(loss) - want) <= 2e-6 * abs(want) + 1e-12
    want_g = 3.0 * 2.0 * ref_d / n
    assert float((p.grad.cpu().double() - want_g).abs().max()) <= 2e-6 * float(want_g.abs().max())
    assert float(ops.mse(p.detach(), t)) == float(loss)


@pytest.mark.gpu
@pytest.mark.parametrize('value', [0.0, 1234.75, 3.0e9, 5.0e9])
def test_ebops_finish_scalar_tail(dev, value):
    """ebops * factor -> uint32 variable and loss term ebops * beta (reference src/hgq/layers/core/base.py:101-104);
    5e9 wraps modulo 2**32 like the reference's cast chain."""
    from hgq2_amd import ops

    e = torch.tensor(value, device=dev, requires_grad=True)
    beta = torch.tensor(3.5e-6, device=dev)
    var = torch.zeros((), dtype=torch.uint32, device=dev)
    out = ops.ebops_finish(e, 0.5, beta, var)
    out.backward(torch.tensor(2.0, device=dev))
    ef = np.float32(value) * np.float32(0.5)
    assert out.item() == float(ef * np.float32(3.5e-6))
    assert int(var.view(torch.int32).item()) & 0xFFFFFFFF == int(ef) & 0xFFFFFFFF
    assert e.grad.item() == float(np.float32(2.0) * np.float32(3.5e-6) * np.float32(0.5))


@pytest.mark.gpu
def test_scalar_loss_terms_summed_in_one_launch():
    """ops.sum_scalars == the chain of additions it stands for, bit for bit, and hands the upstream gradient to
    every term; train.model_loss takes that route for GPU scalars."""
    from hgq2_amd import ops

    dev = torch.device('cuda:0')
    g = torch.Generator().manual_seed(5)
    vals = (torch.randn(70, generator=g) * torch.logspace(-6, 3, 70)).to(dev)
    terms = [vals[t].clone().requires_grad_(t % 3 != 1) for t in range(70)]
    terms[4] = terms[4].detach().reshape(1, 1).requires_grad_(True)
    want = terms[0]
    for t in terms[1:]:
        want = want + t.reshape(())
    got = ops.sum_scalars(terms)
    assert torch.equal(got.reshape(()), want.detach().reshape(()))
    (got * 3.0).backward()
    for t, term in enumerate(terms):
        if term.requires_grad:
            assert term.grad.shape == term.shape and float(term.grad.reshape(())) == 3.0
        else:
            assert term.grad is None


@pytest.mark.gpu
def test_weight_quantizers_in_one_launch_change_nothing():
    """With the kernel / bias quantizers of a model batched ahead of the forward pass (quantizer/prefetch.py) a
    training step gives the same loss and the same gradients, bit for bit, as with one launch per quantizer."""
    import hgq2_amd.core as core
    from hgq2_amd import ops, train
    from hgq2_amd.quantizer.prefetch import prefetch_weight_quantizers
    from hgq2_amd.utils import models

    dev = torch.device('cuda:0')
    results = []
    for flag in (True, False):
        torch.manual_seed(3)
        model = models.mha_block(device=dev)
        x = torch.randn(8, 64, 64, generator=torch.Generator().manual_seed(1)).to(dev)
        with torch.no_grad():
            model(x, training=True)  # build
        core.PREFETCH_WEIGHT_QUANTIZERS = flag
        try:
            y = model(x, training=True)
            loss = train.model_loss(model, (y * y).mean())
            loss.backward()
        finally:
            core.PREFETCH_WEIGHT_QUANTIZERS = True
        results.append((loss.detach().clone(), {n: p.grad.clone() for n, p in model.named_parameters() if p.grad is not None}))
        if flag:
            assert prefetch_weight_quantizers(model) >= 4  # at least the kernels of the q, k, v and output projections
    (l1, g1), (l0, g0) = results
    assert torch.equal(l1, l0) and g1.keys() == g0.keys()
    for n in g1:
        assert torch.equal(g1[n], g0[n]), n


@pytest.mark.gpu
def test_batched_quantizer_matches_single_launches():
    from hgq2_amd import _lib, ops

    dev = torch.device('cuda:0')
    g = torch.Generator().manual_seed(9)
    cases = [(4096, 'RND', 'SAT_SYM', True), (64, 'TRN', 'SAT', False), (33, 'RND_CONV', 'SAT', True), (700, 'RND', 'WRAP', False)]
    xs, ks, is_, fs, modes, singles = [], [], [], [], [], []
    for n, rm, om, kbi in cases:
        x = (torch.randn(n, generator=g) * 3).to(dev).requires_grad_(True)
        k = torch.randint(0, 2, (n,), generator=g).to(torch.uint8).to(dev)
        i = torch.randint(-1, 3, (n,), generator=g).float().to(dev).requires_grad_(True)
        f = (torch.randint(1, 6, (n,), generator=g).float() + (i.detach().cpu() if kbi else 0)).to(dev).requires_grad_(True)
        mode = _lib.mode_bits(rm, om, training=True, kbi=kbi, round_params=True)
        xs.append(x), ks.append(k), is_.append(i), fs.append(f), modes.append(mode)
    ups = [torch.randn(x.shape, generator=g).to(dev) for x in xs]
    ys = ops.quantize_multi(xs, ks, is_, fs, modes)
    sum((y * u).sum() for y, u in zip(ys[:-1], ups)).backward()  # the last output stays unused: zero gradients
    got = [(y.detach(), x.grad, i.grad, f.grad) for y, x, i, f in zip(ys, xs, is_, fs)]
    for t, (x, k, i, f, mode, u) in enumerate(zip(xs, ks, is_, fs, modes, ups)):
        x1, i1, f1 = (v.detach().clone().requires_grad_(True) for v in (x, i, f))
        y1, _, _ = ops.quantize(x1, k, i1, f1, mode)
        assert torch.equal(got[t][0], y1.detach())
        if t < len(xs) - 1:
            (y1 * u).sum().backward()
            for a, b in zip(got[t][1:], (x1.grad, i1.grad, f1.grad)):
                assert torch.equal(a, b)
        else:
            for a in got[t][1:]:
                assert a is None or not a.any()


@pytest.mark.parametrize('kind', ['mlp', 'particle', 'conv', 'mha'])
def test_gradient_sink_gives_the_autograd_update(dev, kind, monkeypatch):
    """``opt.backward(loss)`` leaves the EBOPs gradients of the bit-width variables on the variables and the update
    kernel adds them; the result must be the update of plain ``loss.backward()``.  Where a variable has one piece from
    autograd and one from an EBOPs term the two paths add the same two numbers: bit-identical."""
    from hgq2_amd import ops
    from hgq2_amd.train import SGD, model_loss
    from hgq2_amd.utils import models

    g = torch.Generator().manual_seed(61)
    if kind == 'mlp':
        x, y = torch.randn(4096, 16, generator=g), torch.randint(0, 5, (4096,), generator=g)
        build = lambda: models.qdense_mlp(device=dev)  # noqa: E731
        loss_fn = lambda out: ops.sparse_ce(out, y.to(dev))  # noqa: E731
    elif kind == 'particle':
        x, y = torch.randn(256, 16, 16, generator=g), torch.randint(0, 5, (256,), generator=g)
        build = lambda: models.particle_mlp(n_particles=16, device=dev)  # noqa: E731
        loss_fn = lambda out: ops.sparse_ce(out, y.to(dev))  # noqa: E731
    elif kind == 'conv':
        x, y = torch.rand(64, 28, 28, 1, generator=g), torch.randint(0, 10, (64,), generator=g)
        build = lambda: models.conv_stack(device=dev)  # noqa: E731
        loss_fn = lambda out: ops.sparse_ce(out, y.to(dev))  # noqa: E731
    else:
        x = torch.randn(64, 64, 64, generator=g)
        build = lambda: models.mha_block(device=dev)  # noqa: E731
        loss_fn = lambda out: ops.mse(out)  # noqa: E731
    xd = x.to(dev)
    torch.manual_seed(7)
    a = build()
    a(xd, training=True)
    torch.manual_seed(7)
    b = build()
    b(xd, training=True)
    b.load_state_dict(a.state_dict())
    opt_a, opt_b = SGD(a.parameters(), lr=0.05, fold_regularizers=True), SGD(b.parameters(), lr=0.05, fold_regularizers=True)
    joined = []  # slice sets per joint reduction launch (with the kernel / bias quantizers' backward inside it where it applies)
    plain_reduce, quant_reduce = ops.reduce_slices_multi_op, ops.reduce_slices_quant_multi_op
    monkeypatch.setattr(ops, 'reduce_slices_multi_op', lambda sl, outs, skip: (joined.append(len(sl)), plain_reduce(sl, outs, skip))[1])
    monkeypatch.setattr(ops, 'reduce_slices_quant_multi_op', lambda sl, *a: (joined.append(len(sl)), quant_reduce(sl, *a))[1])
    for step in range(2):
        opt_a.zero_grad()
        la = model_loss(a, loss_fn(a(xd, training=True)), True)
        la.backward()
        opt_a.step()
        opt_b.zero_grad()
        lb = model_loss(b, loss_fn(b(xd, training=True)), True)
        opt_b.backward(lb)
        n_pieces = sum(len(getattr(p, '_hgq_side', None) or ()) for p in b.parameters())
        assert n_pieces > 0, 'no EBOPs gradient took the side channel'
        opt_b.step()
        assert abs(float(la) - float(lb)) <= 1e-6 * abs(float(la))  # the loss value is summed with atomics
        for (name, pa), (_, pb) in zip(a.named_parameters(), b.named_parameters()):
            if kind == 'mlp':
                assert torch.equal(pa, pb), f'{name} step {step}'
            else:
                assert torch.allclose(pa, pb, rtol=1e-6, atol=1e-9), f'{name} step {step}: {float((pa - pb).abs().max()):.3e}'
    if kind in ('mlp', 'mha'):
        # the dense backward of every layer left its slices for one joint reduction per step; in the attention model the
        # output quantizers of the three input projections (bit-widths shared along the batch) add theirs
        assert joined == ([4, 4] if kind == 'mlp' else [7, 7]), joined


def test_dense_backward_in_two_halves_gives_the_same_bits(dev):
    """``qdense_bwd_slices`` + ``reduce_slices_multi`` (several sets per launch, a skipped bias segment, widths that are
    not multiples of 64) against ``qdense_bwd``: identical bits."""
    from hgq2_amd import _lib, ops

    g = torch.Generator().manual_seed(5)
    cases = [(1000, 16, 64, 1, True), (4096, 64, 32, 2, True), (333, 32, 5, 0, False), (64, 8, 4, 1, True)]
    mode = _lib.RND | (_lib.WRAP << 4) | _lib.MODE_TRAINING | _lib.MODE_ROUND_PARAMS
    want, slices, outs, skip = [], [], [], []
    for rows, K, N, bw_rows, has_bias in cases:
        rows -= rows % max(bw_rows, 1)
        x = (torch.randn(rows, K, generator=g) * 3).to(dev)
        qw = (torch.randint(-8, 9, (K, N), generator=g) / 4.0).to(dev)
        y = torch.randn(rows, N, generator=g).to(dev)
        dy = torch.randn(rows, N, generator=g).to(dev)
        f_in = torch.randint(0, 5, (bw_rows * K,), generator=g).float().to(dev)
        act = _lib.ACT_RELU if N > 4 else _lib.ACT_NONE
        m = mode if bw_rows else 0
        want.append(ops.qdense_bwd(dy, y, x, f_in, qw, has_bias, act, m, bw_rows))
        dx, ws = ops.qdense_bwd_slices(dy, y, x, f_in, qw, has_bias, act, m, bw_rows)
        assert torch.equal(dx, want[-1][0])
        slices.append(ws)
        outs += [torch.full((K, N), 7.0, device=dev), torch.full((N,), 7.0, device=dev), torch.full((bw_rows * K,), 7.0, device=dev)]
        skip += [False, not has_bias, False]
    ops.reduce_slices_multi_op(slices, outs, skip)
    for t, (rows, K, N, bw_rows, has_bias) in enumerate(cases):
        dqw, dqb, df = outs[3 * t:3 * t + 3]
        assert torch.equal(dqw, want[t][1]), t
        assert torch.equal(dqb, want[t][2]) if has_bias else bool((dqb == 7.0).all()), t  # a skipped segment is left alone
        assert torch.equal(df, want[t][3]), t
    with pytest.raises(ValueError):
        ops.reduce_slices_multi_op(slices[:1], outs[:2] + [outs[5]], skip[:3])  # lengths do not add up to the width


def test_fused_stack_sees_updates_made_by_the_per_layer_optimizer(dev):
    """Alternating the whole-step kernels with the per-layer path: the fused trainer must not reuse the quantized
    weight image of its previous step after ``SGD.step`` (which writes through ``.data``) changed the variables."""
    from hgq2_amd import ops
    from hgq2_amd.train import SGD, FusedQDenseStack, model_loss
    from hgq2_amd.utils.models import qdense_mlp

    g = torch.Generator().manual_seed(71)
    x, y = torch.randn(2048, 16, generator=g).to(dev), torch.randint(0, 5, (2048,), generator=g).to(dev)
    src = ref.RefMLP(seed=9)
    models = [qdense_mlp(device=dev) for _ in range(2)]
    for m in models:
        _copy_mlp(src, m, dev)
    fused = [FusedQDenseStack(m, lr=0.01) for m in models]
    opts = [SGD(m.parameters(), lr=0.5, fold_regularizers=True) for m in models]
    for f in fused:
        f.step(x, y)
    for step in range(3):
        for m, opt in zip(models, opts):  # a large per-layer update in between
            opt.zero_grad()
            opt.backward(model_loss(m, ops.sparse_ce(m(x, training=True), y), True))
            opt.step()
        fused[1].invalidate()  # the second one quantizes again whatever it believes
        la, lb = fused[0].step(x, y), fused[1].step(x, y)
        # (the reported loss is a sum of some eighty terms added with atomics: equal up to the order of those fp32 adds)
        assert abs(float(la) - float(lb)) <= 5e-6 * abs(float(lb)), f'loss step {step}'
        for pa, pb in zip(models[0].parameters(), models[1].parameters()):
            assert torch.equal(pa, pb), f'step {step}'


def test_beta_written_by_the_controllers_reaches_the_device_loss_term(dev):
    """``BetaScheduler`` / ``BetaPID`` assign the layers' ``beta`` between steps (reference
    src/hgq/utils/sugar/beta_scheduler.py:21-27, beta_pid.py:49-60).  The kernels read beta through the variable's
    device address: the EBOPs * beta term of the loss and the bit-width gradients must follow on the per-layer path, in
    a HIP graph recorded before the change, and in the whole-step kernels."""
    from hgq2_amd import ops
    from hgq2_amd.train import SGD, FusedQDenseStack, GraphedTrainStep, model_loss
    from hgq2_amd.utils.models import qdense_mlp
    from hgq2_amd.utils.sugar import BetaPID, BetaScheduler, FreeEBOPs, PieceWiseSchedule

    g = torch.Generator().manual_seed(72)
    x, y = torch.randn(2048, 16, generator=g).to(dev), torch.randint(0, 5, (2048,), generator=g).to(dev)
    src = ref.RefMLP(seed=10)
    eager, graphed, whole = (qdense_mlp(device=dev) for _ in range(3))
    for m in (eager, graphed, whole):
        _copy_mlp(src, m, dev)
    warm = 2
    opt = SGD(eager.parameters(), lr=0.01, fold_regularizers=True)
    fused = FusedQDenseStack(whole, lr=0.01)

    def eager_step():
        opt.zero_grad()
        loss = model_loss(eager, ops.sparse_ce(eager(x, training=True), y), True)
        loss.backward()
        opt.step()
        return loss.detach()

    for _ in range(warm):  # the capture below trains `warm` steps on its example batch: same history everywhere
        eager_step()
        fused.step(x, y)
    gstep = GraphedTrainStep(graphed, ops.sparse_ce, SGD(graphed.parameters(), lr=0.01, fold_regularizers=True), x, y, warmup=warm)
    gstep()
    eager_step()
    fused.step(x, y)

    schedule = PieceWiseSchedule([(0, 1e-6, 'log'), (2, 1e-2, 'constant')])
    cbs = [BetaScheduler(schedule) for _ in range(3)]
    logger = FreeEBOPs()
    logger.set_model(eager)
    for cb, m in zip(cbs, (eager, graphed, whole)):
        cb.set_model(m)
    terms = []
    for epoch in range(4):
        for cb in cbs:
            cb.on_epoch_begin(epoch, {})
        beta = schedule(epoch)
        assert all(abs(float(layer._beta) - beta) <= 1e-7 * beta for layer in graphed.layers)
        # the whole-step kernels report the full loss; the other two fold the MonoL1 terms into the update and leave
        # them out of the reported value
        with torch.no_grad():
            reg = float(sum(p.regularizer(p) for p in eager.parameters() if getattr(p, 'regularizer', None) is not None and p.requires_grad))
        le, lg, lw = eager_step(), gstep(), fused.step(x, y)
        torch.cuda.synchronize()
        lw = lw - reg
        assert abs(float(lg) - float(le)) <= 2e-6 * abs(float(le)), f'graph replay, epoch {epoch}: {float(lg)} vs {float(le)}'
        assert abs(float(lw) - float(le)) <= 2e-5 * abs(float(le)), f'whole-step kernels, epoch {epoch}: {float(lw)} vs {float(le)}'
        logs = {}
        logger.on_epoch_end(epoch, logs)
        # the loss holds sum(ebops) * beta: compare with the counters the logger reads (state after the update, so loosely)
        with torch.no_grad():
            ce = float(ops.sparse_ce(eager(x, training=False), y))
        terms.append((beta, logs['ebops'], float(le)))
        for (_, pe), (name, pg) in zip(eager.named_parameters(), graphed.named_parameters()):
            assert torch.allclose(pe, pg, rtol=1e-5, atol=1e-7), f'{name} epoch {epoch}'
    # beta rose by four orders of magnitude: the regularisation part of the loss must have risen with it
    reg_first, reg_last = terms[0][0] * terms[0][1], terms[-1][0] * terms[-1][1]
    assert reg_last > 1e3 * reg_first
    assert terms[-1][2] - terms[0][2] > 0.5 * (reg_last - reg_first)
    # a PID controller reads the device counters and writes beta
    pid = BetaPID(target_ebops=0.5 * terms[-1][1], init_beta=1e-5, warmup=0, p=1.0, i=0.1)
    pid.set_model(graphed)
    pid.on_train_begin({})
    pid.on_epoch_begin(0, {})
    before = float(graphed.layers[0]._beta)
    pid.on_epoch_end(0, {})
    pid.on_epoch_begin(1, {})
    after = float(graphed.layers[0]._beta)
    assert after > before > 0  # above the target: beta is pushed up
    l1 = gstep()
    assert torch.isfinite(l1)


@pytest.mark.parametrize('kind', ['mlp', 'particle', 'conv', 'mha'])
def test_saved_and_loaded_model_gives_equal_outputs(dev, kind, tmp_path):
    """The reference's serialization test (tests/base.py:184-201): train a little, calibrate, save, load into a model
    rebuilt from the saved configuration, compare the inference outputs for equality.  Container: ``.npz`` keyed by
    variable path (``hgq2_amd.saving``); the load must also restore what a checkpoint is for - continuing to train gives
    the same next step."""
    from hgq2_amd import ops, saving
    from hgq2_amd.train import SGD, model_loss
    from hgq2_amd.utils import models

    g = torch.Generator().manual_seed(81)
    torch.manual_seed(81)
    if kind == 'mlp':
        x, model = torch.randn(512, 16, generator=g), models.qdense_mlp(device=dev)
    elif kind == 'particle':
        x, model = torch.randn(128, 16, 16, generator=g), models.particle_mlp(n_particles=16, device=dev)
    elif kind == 'conv':
        x, model = torch.rand(32, 28, 28, 1, generator=g), models.conv_stack(device=dev)
    else:
        x, model = torch.randn(32, 64, 64, generator=g), models.mha_block(device=dev)
    xd = x.to(dev)

    def train_step(m):
        opt = SGD(m.parameters(), lr=0.05, fold_regularizers=True)
        opt.zero_grad()
        out = m(xd, training=True)
        opt.backward(model_loss(m, ops.mse(out), True))
        opt.step()

    for _ in range(2):
        train_step(model)
    file = tmp_path / f'{kind}.npz'
    saving.save_model(model, file)
    clone = saving.load_model(file, device=dev)
    with torch.no_grad():
        want, got = model(xd, training=False), clone(xd, training=False)
    assert torch.equal(got, want)
    for (na, ta), (nb, tb) in zip(saving.variable_paths(model).items(), saving.variable_paths(clone).items()):
        assert na == nb and ta.dtype == tb.dtype
        assert torch.equal(ta.view(torch.int32) if ta.dtype == torch.uint32 else ta, tb.view(torch.int32) if tb.dtype == torch.uint32 else tb), na
    train_step(model)
    train_step(clone)
    for (na, ta), (_, tb) in zip(saving.variable_paths(model).items(), saving.variable_paths(clone).items()):
        if ta.dtype == torch.float32:
            assert torch.allclose(ta, tb, rtol=1e-6, atol=1e-9), f'{na} after one more step'


def test_train_step_for_picks_the_path_and_both_paths_agree(dev):
    """`train_step_for` runs a plain QDense stack with cross-entropy on the whole-step kernels and everything else on the
    per-layer operators replayed from a HIP graph; the two paths restate the same sequence, so from the same start state
    they reach the same variables (tracked integer bits and EBOPs exactly, trained variables to the order of fp32
    sums)."""
    import io

    from hgq2_amd import saving
    from hgq2_amd.config import LayerConfigScope, QuantizerConfigScope
    from hgq2_amd.core import Sequential
    from hgq2_amd.layers import QDense
    from hgq2_amd.train import train_step_for

    g = torch.Generator().manual_seed(5)
    torch.manual_seed(5)
    x = torch.randn(1000, 12, generator=g).to(dev)
    labels = torch.randint(0, 4, (1000,), generator=g).to(dev)

    def stack(widths, **kw):
        with QuantizerConfigScope(place='all', default_q_type='kbi', overflow_mode='SAT_SYM'), \
                QuantizerConfigScope(place='datalane', default_q_type='kif', overflow_mode='WRAP'), \
                LayerConfigScope(enable_ebops=True, beta0=1e-5):
            model = Sequential([QDense(w, activation='relu' if n + 1 < len(widths) else None, **kw) for n, w in enumerate(widths)])
        model(x, training=True)
        return model

    model = stack([24, 16, 4])
    buf = io.BytesIO()
    saving.save_model(model, buf)
    buf.seek(0)
    clone = saving.load_model(buf, device=dev)
    fused = train_step_for(model, x, labels, lr=0.05)
    layered = train_step_for(clone, x, labels, lr=0.05, fused=False)
    assert fused.path == 'fused' and layered.path == 'layers_graph'
    buf.seek(0)
    saving.load_weights(clone, buf)  # the capture's warm-up steps moved the clone: back to the common start
    for step in range(4):
        fused(x, labels), layered(x, labels)  # (the loss values differ by the regularizer terms the per-layer update folds in)
        for a, b in zip(model.layers, clone.layers):
            assert torch.equal(a.iq.quantizer._i, b.iq.quantizer._i)
            assert int(a._ebops.view(torch.int32)) == int(b._ebops.view(torch.int32))
        for (name, pa), (_, pb) in zip(model.named_parameters(), clone.named_parameters()):
            err = (pa.detach().double() - pb.detach().double()).abs().max().item()
            assert err <= 2e-5 * (pb.detach().abs().max().item() + 1e-6), (step, name, err)

    # outside the whole-step kernels' cover: a layer wider than 64, an output quantizer, another loss
    assert train_step_for(stack([80, 4]), x, labels).path == 'layers_graph'
    assert train_step_for(stack([16, 4], enable_oq=True), x, labels).path == 'layers_graph'
    target = torch.randn(1000, 4, generator=g).to(dev)
    assert train_step_for(stack([16, 4]), x, target, loss='mse').path == 'layers_graph'
    with pytest.raises(ValueError):
        train_step_for(stack([80, 4]), x, labels, fused=True)


@pytest.mark.parametrize('kind', ['dense_relu', 'einsum', 'einsum_small_table'])
def test_output_quantizer_inside_the_dense_kernel(dev, kind):
    """A layer's output quantizer of the fusable kind (plain KIF, WRAP, training) runs inside the contraction kernel.
    The same layer with the bf16-part kernels switched off takes the separate launches: outputs, tracked integer bits of
    both quantizers and EBOPs agree bit for bit (operands of a few bits: the contraction is exact either way), gradients
    to the order of fp32 sums."""
    import io

    from hgq2_amd import _lib, ops, saving
    from hgq2_amd.config import LayerConfigScope, QuantizerConfigScope
    from hgq2_amd.core import Sequential
    from hgq2_amd.layers import QDense, QEinsumDense
    from hgq2_amd.train import SGD, model_loss

    lib = _lib.load()
    g = torch.Generator().manual_seed(3)
    torch.manual_seed(3)
    with QuantizerConfigScope(place='all', default_q_type='kbi', overflow_mode='SAT_SYM'), \
            QuantizerConfigScope(place='datalane', default_q_type='kif', overflow_mode='WRAP'), \
            LayerConfigScope(enable_ebops=True, beta0=1e-5):
        if kind == 'dense_relu':
            x = torch.randn(300, 24, generator=g)
            layers = [QDense(32, activation='relu', enable_oq=True), QDense(8, enable_oq=True)]
        elif kind == 'einsum':
            x = torch.randn(70, 64, 16, generator=g)
            layers = [QEinsumDense('bpf,fnh->bpnh', (64, 4, 8), bias_axes='nh', enable_oq=True)]
        else:
            x = torch.randn(130, 16, 20, generator=g)
            layers = [QEinsumDense('bpf,fh->bph', (16, 12), bias_axes='h', activation='relu', enable_oq=True)]
    model = Sequential(layers)
    x = x.to(dev)
    model(x, training=True)
    with torch.no_grad():
        for layer in layers:
            f = layer.oq.quantizer._f
            f.add_(torch.randint(-2, 3, f.shape, generator=g).float().to(dev))
    buf = io.BytesIO()
    saving.save_model(model, buf)
    buf.seek(0)
    clone = saving.load_model(buf, device=dev)
    up = torch.randn(model(x, training=False).shape, generator=g).to(dev)
    buf.seek(0)
    saving.load_weights(model, buf)

    def run(m, steps=2):
        opt = SGD(m.parameters(), lr=0.05, fold_regularizers=True)
        outs = []
        for _ in range(steps):
            opt.zero_grad()
            y = m(x, training=True)
            outs.append(y.detach().clone())
            loss = model_loss(m, ops.mse(y * up), True)
            opt.backward(loss)
            opt.step()
        return outs

    launches = []
    real = ops.qdense_fwd_oq

    def spy(*a, **k):
        launches.append(1)
        return real(*a, **k)

    ops.qdense_fwd_oq = spy
    was = lib.hgq_dense_use_bf16_parts(1)  # (the process may have been started on the fp32 matrix instruction)
    try:
        fused = run(model)
        n_fused = len(launches)
        lib.hgq_dense_use_bf16_parts(0)
        plain = run(clone)
    finally:
        lib.hgq_dense_use_bf16_parts(was)
        ops.qdense_fwd_oq = real
    assert n_fused == 2 * len(layers) and len(launches) == n_fused, 'the fused kernel runs exactly where it is switched on'
    for a, b in zip(fused, plain):
        assert torch.equal(a, b)
    for la, lb in zip(model.layers, clone.layers):
        assert torch.equal(la.oq.quantizer._i, lb.oq.quantizer._i) and torch.equal(la.iq.quantizer._i, lb.iq.quantizer._i)
        assert int(la._ebops.view(torch.int32)) == int(lb._ebops.view(torch.int32))
    for (name, pa), (_, pb) in zip(model.named_parameters(), clone.named_parameters()):
        err = (pa.detach().double() - pb.detach().double()).abs().max().item()
        assert err <= 2e-5 * (pb.detach().abs().max().item() + 1e-6), (name, err)

    # plain autograd (no gradient sink): the one-pass backward reduces its own slices and hands every gradient back
    def grads(m):
        for p_ in m.parameters():
            p_.grad = None
        model_loss(m, ops.mse(m(x, training=True) * up)).backward()
        return {n: p_.grad.detach().clone() for n, p_ in m.named_parameters() if p_.grad is not None}

    was = lib.hgq_dense_use_bf16_parts(1)
    try:
        ga = grads(model)
        lib.hgq_dense_use_bf16_parts(0)
        gb = grads(clone)
    finally:
        lib.hgq_dense_use_bf16_parts(was)
    assert ga.keys() == gb.keys() and any('oq' in n and n.endswith('_f') for n in ga)
    for n in ga:
        err = (ga[n].double() - gb[n].double()).abs().max().item()
        assert err <= 2e-5 * (gb[n].abs().max().item() + 1e-6), (n, err)


@pytest.mark.parametrize('rows,row_shape,dtype,batch', [(1000, (16,), torch.float32, 128), (77, (3, 5), torch.float32, 10),
                                                        (300, (7,), torch.int32, 64), (64, (4,), torch.float32, 64)])
def test_batch_feed_draws_the_rows_of_the_order_in_turn(dev, rows, row_shape, dtype, batch):
    """``ops.gather_batch`` (``hgq_gather_batch``): successive launches fill the buffers with rows
    ``order[0:batch]``, ``order[batch:2 batch]``, ... of the samples and the labels, eagerly and as a replayed graph."""
    from hgq2_amd import ops
    from hgq2_amd.train import ResidentBatches

    g = torch.Generator().manual_seed(rows)
    x = (torch.randn((rows,) + row_shape, generator=g) * 100).to(dtype).to(dev)
    y = torch.randint(0, 9, (rows,), generator=g).to(dev)
    feed = ResidentBatches(x, y)
    xb, yb = torch.empty((batch,) + row_shape, dtype=dtype, device=dev), torch.empty(batch, dtype=torch.int64, device=dev)
    for order in (None, torch.randperm(rows, generator=g).to(dev)):
        feed.start_epoch(order)
        idx = torch.arange(rows, device=dev) if order is None else order
        for b in range(rows // batch):
            feed.draw(xb, yb)
            sel = idx[b * batch:(b + 1) * batch]
            assert torch.equal(xb, x[sel]) and torch.equal(yb, y[sel]), (order is None, b)
        assert int(feed.state[0]) == (rows // batch) * batch and int(feed.state[1]) == 0
    # recorded once, replayed: every replay draws the next batch
    feed.start_epoch(None)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        feed.draw(xb, yb)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        feed.draw(xb, yb)
    for b in range(1, rows // batch):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(xb, x[b * batch:(b + 1) * batch]) and torch.equal(yb, y[b * batch:(b + 1) * batch]), b


@pytest.mark.parametrize('fused,shuffle', [(False, False), (None, False), (False, True)])
def test_fit_trains_every_batch_once_on_the_fast_path(dev, fused, shuffle):
    """`train.fit`: epochs of full batches (in the rows' order, or shuffled anew per epoch) through the recorded step - which
    draws its own batches from the data set in device memory - or the whole-step kernels, plus a shorter last
    batch, hooks in Keras' order.  On the per-layer path the variables equal those of the same steps launched one by one,
    bit for bit and the logged losses agree to 1e-6 (a sum on the device against a sum on the host); on the whole-step path
    (same arithmetic restated) the epoch losses agree to 1e-5 and the variables to 1e-4 of their largest entry."""
    from hgq2_amd import ops
    from hgq2_amd.train import SGD, fit, folded_regularizer_loss, model_loss
    from hgq2_amd.utils.models import qdense_mlp
    from hgq2_amd.utils.sugar import BetaScheduler, Callback, FreeEBOPs

    g = torch.Generator().manual_seed(12)
    n, bs = 5 * 512 + 200, 512
    x = torch.randn(n, 16, generator=g).to(dev)
    y = torch.randint(0, 5, (n,), generator=g).to(dev)
    src = ref.RefMLP(seed=6)
    model, twin = qdense_mlp(device=dev), qdense_mlp(device=dev)
    _copy_mlp(src, model, dev), _copy_mlp(src, twin, dev)

    calls = []

    class Spy(Callback):
        def on_train_begin(self, logs=None):
            calls.append('train')

        def on_epoch_begin(self, epoch, logs=None):
            calls.append(f'begin{epoch}')

        def on_epoch_end(self, epoch, logs=None):
            calls.append(f'end{epoch}')

    betas = [1e-5, 3e-5]
    history = fit(model, x, y, lr=0.01, batch_size=bs, epochs=2, shuffle=shuffle, seed=5, fused=fused,
                  callbacks=[Spy(), BetaScheduler(lambda e: betas[e]), FreeEBOPs()])
    assert calls == ['train', 'begin0', 'end0', 'begin1', 'end1']
    assert [h['beta'] for h in history] == betas and all(h['ebops'] > 0 for h in history)

    opt = SGD(twin.parameters(), lr=0.01, fold_regularizers=True)
    want = []
    gen = torch.Generator().manual_seed(5)  # the loop's own generator: one permutation per epoch
    for e in range(2):
        for layer in twin.layers:
            layer._beta.fill_(betas[e])
        total = 0.0
        xe, ye = x, y
        if shuffle:
            order = torch.randperm(n, generator=gen).to(dev)
            xe, ye = x[order], y[order]
        for lo in range(0, n, bs):
            opt.zero_grad()
            with ops.overlap_ebops():
                loss = model_loss(twin, ops.sparse_ce(twin(xe[lo:lo + bs], training=True), ye[lo:lo + bs]), True)
                opt.backward(loss)
                opt.step()
            total += float(loss.detach())
        want.append(total / 6 + folded_regularizer_loss(twin))
    torch.cuda.synchronize()
    for h, w in zip(history, want):
        assert abs(h['loss'] - w) <= (1e-6 if fused is False else 1e-5) * abs(w)
    if fused is False:
        for pm, pt in zip(model.parameters(), twin.parameters()):
            assert torch.equal(pm, pt)
    else:
        for pm, pt in zip(model.parameters(), twin.parameters()):
            scale = pt.abs().max().item() + 1e-6
            assert (pm - pt).abs().max().item() <= 1e-4 * scale
