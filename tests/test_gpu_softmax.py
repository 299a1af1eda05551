"""GPU parity of the one-pass table-softmax kernels (hgq_qsoftmax_fwd / hgq_qsoftmax_bwd):

* against the CPU oracle's restatement of QSoftmax (reference src/hgq/layers/softmax.py) on
  identical bit-widths and inputs, over the row layouts the kernel family covers;
* against the layer's own composed path (one quantizer kernel per stage plus elementwise
  library ops) at the full size of the attention benchmark configuration, where the oracle
  would take minutes: quantized values bit-exact, gradients within 1e-5 relative.
"""

import pytest
import torch

from oracle import twin
from tests.test_gpu_more_layers import _close, _compare_step, readme_scopes

pytestmark = pytest.mark.gpu


def _make(shape, dev, g, *, enable_oq=True, exp_overflow='SAT', scaler=0.25, oq_hom=None):
    from hgq2_amd.config import QuantizerConfig
    from hgq2_amd.layers import QSoftmax

    kw = {}
    if oq_hom is not None:
        kw['oq_conf'] = QuantizerConfig(place='datalane', homogeneous_axis=oq_hom)
    with readme_scopes():
        layer = QSoftmax(axis=-1, enable_oq=enable_oq, input_scaler=scaler,
                         exp_iq_conf=QuantizerConfig(place='datalane', overflow_mode=exp_overflow), **kw)
    x = torch.randn(shape, generator=g) * 3
    layer(x.to(dev), training=True)  # build, adapt the tracked integer bits
    return layer, x


def _named(layer, r, xp, xr):
    e, i, re_, ri = layer.exp_table, layer.inv_table, r.exp_table, r.inv_table
    named_p = [('x', xp), ('exp_iq_f', e.iq.quantizer._f), ('exp_iq_i', e.iq.quantizer._i), ('exp_oq_b', e.oq.quantizer._b),
               ('exp_oq_i', e.oq.quantizer._i), ('inv_iq_f', i.iq.quantizer._f), ('inv_oq_b', i.oq.quantizer._b),
               ('inv_oq_i', i.oq.quantizer._i)]
    named_r = [('x', xr), ('exp_iq_f', re_.iq.quantizer._f), ('exp_iq_i', re_.iq.quantizer._i),
               ('exp_oq_b', re_.oq.quantizer._b), ('exp_oq_i', re_.oq.quantizer._i), ('inv_iq_f', ri.iq.quantizer._f),
               ('inv_oq_b', ri.oq.quantizer._b), ('inv_oq_i', ri.oq.quantizer._i)]
    if layer.enable_oq:
        named_p.append(('oq_f', layer.oq.quantizer._f))
        named_r.append(('oq_f', r.oq.quantizer._f))
    return named_p, named_r


@pytest.mark.parametrize('shape,enable_oq,exp_overflow,oq_hom', [
    ((32, 4, 16, 64), True, 'SAT', None),    # 128-bit accesses, four rows side by side
    ((16, 3, 10), True, 'WRAP', None),       # short rows, table rows that do not tile a wavefront
    ((24, 8, 16), True, 'SAT', None),        # four rows side by side in a wavefront
    ((8, 6, 100), True, 'SAT', None),        # 128-bit accesses, a row spans 32 lanes
    ((4, 8, 200), True, 'WRAP', None),       # 128-bit accesses, a row spans the wavefront
    ((40, 7, 32), False, 'SAT', None),       # no output quantizer
    ((12, 6, 24), True, 'SAT', (0, 1)),      # output quantizer table shared by all rows
])
def test_fused_softmax_matches_oracle(dev, shape, enable_oq, exp_overflow, oq_hom):
    import hgq2_amd.layers.softmax as sm

    g = torch.Generator().manual_seed(11)
    layer, x = _make(shape, dev, g, enable_oq=enable_oq, exp_overflow=exp_overflow, oq_hom=oq_hom)
    assert layer._fused_plan(x.to(dev), True, None) is not None, 'this configuration must take the fused kernel'
    with torch.no_grad():  # heterogeneous output bit-widths
        if enable_oq:
            f = layer.oq.quantizer._f
            f.copy_(torch.randint(3, 9, f.shape, generator=g).float())
    r = twin.ref_softmax(layer)
    xp, xr = x.to(dev).requires_grad_(True), x.clone().requires_grad_(True)
    named_p, named_r = _named(layer, r, xp, xr)
    calls = {'n': 0}
    orig = sm.ops.qsoftmax

    def counting(*a, **k):
        calls['n'] += 1
        return orig(*a, **k)

    sm.ops.qsoftmax = counting
    try:
        _compare_step(layer, r, lambda t: layer(xp, training=t), lambda t: r(xr, training=t), named_p, named_r)
    finally:
        sm.ops.qsoftmax = orig
    assert calls['n'] == 1
    # state: tracked integer bits and the EBOPs variables of the layer and its two tables
    for qp, qr in ((layer.exp_table.iq, r.exp_table.iq), (layer.inv_table.iq, r.inv_table.iq)) + (
            ((layer.oq, r.oq),) if enable_oq else ()):
        assert torch.equal(qp.quantizer._i.cpu(), qr.quantizer._i.detach())
    assert int(layer.exp_table._ebops.cpu().view(torch.int32)) == int(r.exp_table.ebops_value)
    assert int(layer.inv_table._ebops.cpu().view(torch.int32)) == int(r.inv_table.ebops_value)
    assert int(layer._ebops.cpu().view(torch.int32)) == int(r.ebops_value)
    # inference forward (overflow applied, empty words zeroed)
    with torch.no_grad():
        got = layer(x.to(dev), training=False)
        want = r(x, training=False)
    _close(got, want, what='inference output')


def _grads(layer, xp):
    e, i = layer.exp_table, layer.inv_table
    ps = [xp, e.iq.quantizer._f, e.iq.quantizer._i, e.oq.quantizer._b, e.oq.quantizer._i, i.iq.quantizer._f,
          i.oq.quantizer._b, i.oq.quantizer._i, layer.oq.quantizer._f]
    out = [None if p.grad is None else p.grad.detach().clone() for p in ps]
    for p in ps:
        p.grad = None
    return out


def test_fused_softmax_equals_composed_path_at_attention_size(dev):
    """Scores of the attention configuration, [2048, 4, 64, 64], softmax over the last axis with
    input_scaler = 1 / sqrt(16): the fused kernels against the per-stage path of the same layer."""
    import hgq2_amd.layers.softmax as sm

    g = torch.Generator().manual_seed(5)
    shape = (2048, 4, 64, 64)
    layer, x = _make(shape, dev, g, scaler=0.25)
    with torch.no_grad():
        f = layer.oq.quantizer._f
        f.copy_(torch.randint(4, 9, f.shape, generator=g).float())
    state = {n: p.detach().clone() for n, p in layer.state_dict().items()}
    w = torch.randn(shape, generator=g).to(dev)
    results = []
    for fused in (True, False):
        layer.load_state_dict(state)
        sm.FUSED = fused
        try:
            xp = x.to(dev).requires_grad_(True)
            y = layer(xp, training=True)
            (y * w).sum().backward()
        finally:
            sm.FUSED = True
        i_vars = [q.quantizer._i.detach().clone() for q in (layer.exp_table.iq, layer.inv_table.iq, layer.oq)]
        results.append((y.detach(), _grads(layer, xp), i_vars, [float(t.detach()) for t in layer.losses[:3]]))
    (y1, g1, i1, l1), (y2, g2, i2, l2) = results
    assert torch.equal(y1, y2), 'quantized outputs must be bit-identical'
    for a, b in zip(i1, i2):
        assert torch.equal(a, b)
    assert l1 == l2
    names = ['x', 'exp_iq_f', 'exp_iq_i', 'exp_oq_b', 'exp_oq_i', 'inv_iq_f', 'inv_oq_b', 'inv_oq_i', 'oq_f']
    for n, a, b in zip(names, g1, g2):
        assert (a is None) == (b is None), n
        if a is None:
            continue
        scale = b.abs().max().item() + 1e-12
        # sums over 33.5 M terms are accumulated in different orders: fp32 summation noise only
        tol = (1e-5 if n in ('x', 'oq_f') else 2e-4) * scale
        assert float((a - b).abs().max()) <= tol, f'grad {n}: {float((a - b).abs().max()):.3e} vs scale {scale:.3e}'
