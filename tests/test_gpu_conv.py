"""GPU parity of the implicit-GEMM convolution kernels (hgq_conv2d_fwd / hgq_conv2d_bwd) against
the library routine they reduce to, evaluated in fp64 on the CPU: forward values and all three
gradients within 1e-5 relative; exact where the operands are small integers (the EBOPs use)."""

import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu


def _ref_conv(x, w, b, strides, padding, dilation, relu):
    """Channels-last reference in fp64; 'same' pads like Keras (odd pad after)."""
    x = x.double().permute(0, 3, 1, 2)
    wt = w.double().permute(3, 2, 0, 1)
    if padding == 'same':
        pads = []
        for d in (1, 0):
            n, k, s, dl = x.shape[2 + d], w.shape[d], strides[d], dilation[d]
            total = max((-(-n // s) - 1) * s + dl * (k - 1) + 1 - n, 0)
            pads += [total // 2, total - total // 2]
        x = F.pad(x, pads)
    y = F.conv2d(x, wt, None if b is None else b.double(), strides, 0, dilation).permute(0, 2, 3, 1)
    return torch.relu(y) if relu else y


CASES = [
    # B, H, W, C, kh, kw, F, strides, padding, dilation, relu, bias
    (1024 // 16, 28, 28, 1, 3, 3, 32, (1, 1), 'valid', (1, 1), True, True),    # first layer of the image configuration
    (16, 13, 13, 32, 3, 3, 32, (1, 1), 'valid', (1, 1), True, True),           # second layer
    (5, 10, 9, 3, 3, 3, 8, (2, 1), 'same', (1, 1), True, True),
    (3, 12, 11, 5, 2, 4, 40, (1, 2), 'same', (1, 1), False, False),            # more than 32 filters: 64-wide tiles
    (2, 9, 14, 40, 3, 3, 70, (2, 2), 'valid', (1, 1), True, True),             # more than 32 channels in the data gradient
    (4, 11, 11, 6, 3, 3, 10, (1, 1), 'same', (2, 2), False, True),             # dilation
    (7, 1, 1, 300, 1, 1, 10, (1, 1), 'valid', (1, 1), False, True),            # dense as 1 x 1
    (0, 5, 5, 3, 3, 3, 4, (1, 1), 'valid', (1, 1), True, True),                # empty batch
    (6, 9, 9, 2, 3, 3, 10, (1, 1), 'same', (1, 1), True, True),                # few channels, filters not a multiple of 4
    (48, 1, 1, 3872, 1, 1, 10, (1, 1), 'valid', (1, 1), True, True),           # long contraction, few rows: split along k
    (300, 6, 6, 2, 3, 3, 24, (1, 1), 'valid', (1, 1), True, True),             # K = 18: row-split weight gradient
    (40, 8, 8, 5, 3, 3, 16, (1, 1), 'valid', (1, 1), False, True),             # K = 45: two k blocks, two row groups
    (3, 10, 11, 8, 3, 2, 12, (2, 1), 'same', (1, 2), True, True),              # 128-bit gathers with stride, dilation, padding
    (2, 9, 9, 36, 3, 3, 36, (2, 2), 'same', (1, 1), True, True),               # 128-bit gathers, 64-wide tiles both ways
    (1024, 12, 12, 8, 3, 3, 8, (1, 1), 'valid', (1, 1), True, True),           # more row tiles than workgroups
    (5, 40, 37, 3, 3, 3, 32, (1, 1), 'same', (1, 1), True, True),              # few channels: ragged pixel tiles both ways, padding
    (3, 19, 70, 4, 3, 3, 16, (1, 1), 'valid', (1, 1), False, True),            # four channels
    (4, 17, 33, 1, 5, 5, 7, (1, 1), 'same', (1, 1), True, False),              # 5 x 5 on one channel, scalar staging
    (2, 20, 45, 1, 3, 3, 12, (2, 1), 'valid', (2, 3), True, True),             # few channels forward with stride and dilation
    (900, 9, 34, 2, 3, 3, 8, (1, 1), 'same', (1, 1), True, True),              # more pixel tiles than workgroups
    (3, 14, 9, 8, 3, 3, 16, (1, 1), 'same', (2, 1), True, True),               # LDS-resident operands: dilation and padding both ways
    (2, 20, 70, 8, 3, 3, 12, (1, 1), 'same', (1, 1), True, True),              # ... several pixel tiles along x and y
    (2, 40, 12, 16, 5, 2, 32, (2, 1), 'valid', (1, 1), False, True),           # ... stride in the forward, 5 x 2 kernel
]


@pytest.mark.parametrize('case', CASES)
def test_conv2d_matches_fp64_reference(dev, case):
    from hgq2_amd import _lib, ops

    B, H, W, C, kh, kw, Fo, strides, padding, dilation, relu, bias = case
    g = torch.Generator().manual_seed(CASES.index(case))
    x = torch.randn(B, H, W, C, generator=g)
    w = torch.randn(kh, kw, C, Fo, generator=g) * 0.3
    b = torch.randn(Fo, generator=g) if bias else None
    xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    br = b.clone().requires_grad_(True) if bias else None
    want = _ref_conv(xr, wr, br, strides, padding, dilation, relu)
    xp, wp = x.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
    bp = b.to(dev).requires_grad_(True) if bias else None
    got = ops.conv2d(xp, wp, bp, strides, padding, dilation, _lib.ACT_RELU if relu else _lib.ACT_NONE)
    assert tuple(got.shape) == tuple(want.shape)
    if B == 0:
        return
    scale = want.abs().max().item() + 1e-9
    assert float((got.detach().cpu().double() - want.detach()).abs().max()) <= 1e-5 * scale
    up = torch.randn(want.shape, generator=g)
    if relu:
        # An output within fp32 rounding of the kink has no agreed derivative: fp32 and fp64 may
        # land on opposite sides of zero there, so such outputs get no upstream gradient.
        pre = _ref_conv(x, w, b, strides, padding, dilation, False)
        up = up * (pre.abs() > 1e-5 * scale)
    (want * up.double()).sum().backward()
    (got * up.to(dev)).sum().backward()
    # every gradient entry is a sum of products: bound its error by 1e-5 of the sum of the |products|, which the same
    # reference gives when it is run on the absolute values (without the activation, its mask folded into the upstream gradient)
    xa, wa = x.abs().requires_grad_(True), w.abs().requires_grad_(True)
    ba = b.abs().requires_grad_(True) if bias else None
    dz = up.double() * (want.detach() > 0) if relu else up.double()
    (_ref_conv(xa, wa, ba, strides, padding, dilation, False) * dz.abs()).sum().backward()
    for name, p, r, a in (('x', xp, xr, xa), ('w', wp, wr, wa)) + ((('b', bp, br, ba),) if bias else ()):
        err = (p.grad.cpu().double() - r.grad.double()).abs()
        tol = 1e-5 * a.grad.double() + 1e-30
        assert bool((err <= tol).all()), f'grad {name}: {float((err / tol).max()):.2f} x the bound of 1e-5 of the summed |terms|'


WGRAD_PATCH_CASES = [
    # B, H, W, C, kh, F, padding, bits of the source (0: arbitrary fp32), misaligned source
    (9, 13, 13, 32, 3, 32, 'valid', 6, False),    # the image configuration's second layer: one bf16 part per source value
    (9, 13, 13, 32, 3, 32, 'valid', 14, False),   # two parts
    (9, 13, 13, 32, 3, 32, 'valid', 0, False),    # three parts
    (700, 9, 10, 8, 3, 20, 'same', 5, False),     # more images than workgroups, padding, filters not a multiple of 32
    (3, 50, 41, 16, 3, 12, 'same', 7, False),     # several bands per image, the last one short
    (4, 18, 15, 12, 5, 28, 'same', 6, False),     # 5 x 5, channels not a multiple of 8
    (3, 12, 12, 24, 5, 8, 'valid', 0, False),
    (5, 13, 13, 32, 3, 32, 'valid', 6, True),     # a source that is not 16-byte aligned keeps the slice count: gathered kernels
]


@pytest.mark.parametrize('case', WGRAD_PATCH_CASES)
def test_weight_gradient_from_lds_patches(dev, case):
    """Kernel / bias gradient of 3 x 3 and 5 x 5 layers with up to 32 channels and filters (both operands of a band of an
    image staged once in LDS, dz as bf16 parts): against the fp64 reference, error bound 1e-5 of the summed |terms|."""
    from hgq2_amd import _lib, ops

    B, H, W, C, k, Fo, padding, bits, misaligned = case
    g = torch.Generator().manual_seed(WGRAD_PATCH_CASES.index(case))
    if bits:
        x = torch.randint(-(1 << (bits - 1)), 1 << (bits - 1), (B, H, W, C), generator=g).float() / 16.0
    else:
        x = torch.randn(B, H, W, C, generator=g)
    w = torch.randn(k, k, C, Fo, generator=g) * 0.3
    b = torch.randn(Fo, generator=g)
    xr, wr, br = x.clone().requires_grad_(True), w.clone().requires_grad_(True), b.clone().requires_grad_(True)
    want = _ref_conv(xr, wr, br, (1, 1), padding, (1, 1), True)
    if misaligned:
        xp = torch.zeros(x.numel() + 1, device=dev)[1:].view(x.shape).copy_(x.to(dev)).requires_grad_(True)
        assert xp.data_ptr() % 16 != 0
    else:
        xp = x.to(dev).requires_grad_(True)
    wp, bp = w.to(dev).requires_grad_(True), b.to(dev).requires_grad_(True)
    got = ops.conv2d(xp, wp, bp, (1, 1), padding, (1, 1), _lib.ACT_RELU)
    scale = want.abs().max().item() + 1e-9
    up = torch.randn(want.shape, generator=g)
    pre = _ref_conv(x, w, b, (1, 1), padding, (1, 1), False)
    up = up * (pre.abs() > 1e-5 * scale)
    (want * up.double()).sum().backward()
    (got * up.to(dev)).sum().backward()
    xa, wa, ba = x.abs().requires_grad_(True), w.abs().requires_grad_(True), b.abs().requires_grad_(True)
    dz = up.double() * (want.detach() > 0)
    (_ref_conv(xa, wa, ba, (1, 1), padding, (1, 1), False) * dz.abs()).sum().backward()
    for name, p_, r, a in (('w', wp, wr, wa), ('b', bp, br, ba), ('x', xp, xr, xa)):
        err = (p_.grad.cpu().double() - r.grad.double()).abs()
        tol = 1e-5 * a.grad.double() + 1e-30
        assert bool((err <= tol).all()), f'grad {name}: {float((err / tol).max()):.2f} x the bound of 1e-5 of the summed |terms|'


def test_conv2d_small_integers_exact(dev):
    """Bit-width tensors convolved for EBOPs hold small integers: products and sums are exact in fp32."""
    from hgq2_amd import ops

    g = torch.Generator().manual_seed(3)
    x = torch.randint(0, 12, (1, 28, 28, 4), generator=g).float()
    w = torch.randint(0, 9, (3, 3, 4, 32), generator=g).float()
    got = ops.conv2d(x.to(dev), w.to(dev), None)
    want = _ref_conv(x, w, None, (1, 1), 'valid', (1, 1), False)
    assert torch.equal(got.cpu().double(), want)


def test_wide_dense_layer_matches_oracle(dev):
    """QDense 3872 -> 10 (the classifier of the image configuration): beyond the fused dense
    kernels, so the contraction runs in the 1 x 1 implicit-GEMM kernels."""
    from hgq2_amd.layers import QDense
    from oracle import twin
    from tests.test_gpu_more_layers import _compare_step, _perturb, readme_scopes

    g = torch.Generator().manual_seed(9)
    with readme_scopes():
        layer = QDense(10)
    x = torch.rand(64, 3872, generator=g)
    layer(x.to(dev), training=True)
    _perturb(layer, g)
    r = twin.ref_dense(layer)
    xp, xr = x.to(dev).requires_grad_(True), x.clone().requires_grad_(True)
    named_p = [('x', xp), ('kernel', layer._kernel), ('bias', layer.bias), ('iq_f', layer.iq.quantizer._f),
               ('kq_b', layer.kq.quantizer._b), ('kq_i', layer.kq.quantizer._i)]
    named_r = [('x', xr), ('kernel', r.kernel), ('bias', r.bias), ('iq_f', r.iq.quantizer._f), ('kq_b', r.kq.quantizer._b),
               ('kq_i', r.kq.quantizer._i)]
    _compare_step(layer, r, lambda t: layer(xp, training=t), lambda t: r(xr, training=t), named_p, named_r)
    assert torch.equal(layer.iq.quantizer._i.cpu(), r.iq.quantizer._i.detach())
    assert int(layer.ebops.cpu().view(torch.int32)) == int(r.ebops_value)


@pytest.mark.parametrize('mode', ['max', 'avg'])
@pytest.mark.parametrize('case', [
    # B, H, W, C, pool, strides, padding
    (16, 26, 26, 32, (2, 2), None, 'valid'),     # the pooling of the image configuration
    (5, 9, 11, 3, (3, 2), (2, 1), 'same'),       # overlapping windows, odd padding, scalar channel path
    (4, 7, 7, 8, (3, 3), (3, 3), 'valid'),       # border pixels that no window covers
    (3, 8, 6, 4, (2, 3), (1, 2), 'same'),
    (2, 7, 8, 4, (3, 3), (3, 3), 'same'),        # disjoint windows that start in the padding
    (2, 9, 10, 1, (2, 2), (3, 3), 'valid'),      # stride larger than the window: gaps between windows
    (3, 7, 9, 8, (2, 2), (2, 2), 'same'),
])
def test_pooling_layers_match_oracle(dev, mode, case):
    """QMaxPooling2D / QAveragePooling2D: values, EBOPs, tracked bits and gradients (incl. where the
    gradient of a tied maximum goes: quantized ReLU-like inputs tie often) against the oracle twin."""
    from hgq2_amd.layers import QAveragePooling2D, QMaxPooling2D
    from oracle import twin
    from tests.test_gpu_more_layers import _compare_step, _perturb, readme_scopes

    B, H, W, C, pool, strides, padding = case
    g = torch.Generator().manual_seed(B + H)
    cls = QMaxPooling2D if mode == 'max' else QAveragePooling2D
    with readme_scopes():
        layer = cls(pool, strides=strides, padding=padding)
    x = torch.relu(torch.randn(B, H, W, C, generator=g))  # many exact zeros after quantization: ties
    layer(x.to(dev), training=True)
    _perturb(layer, g)
    r = twin.ref_pooling2d(layer)
    xp, xr = x.to(dev).requires_grad_(True), x.clone().requires_grad_(True)
    named_p = [('x', xp), ('iq_f', layer.iq.quantizer._f)]
    named_r = [('x', xr), ('iq_f', r.iq.quantizer._f)]
    _compare_step(layer, r, lambda t: layer(xp, training=t), lambda t: r(xr, training=t), named_p, named_r)
    assert torch.equal(layer.iq.quantizer._i.cpu(), r.iq.quantizer._i.detach())
    assert int(layer.ebops.cpu().view(torch.int32)) == int(r.ebops_value)


@pytest.mark.parametrize('case', [(28, 28, 1, 3, 3, 32, (1, 1), 'valid', (1, 1)), (13, 13, 32, 3, 3, 32, (1, 1), 'valid', (1, 1)),
                                  (10, 9, 3, 3, 3, 8, (2, 1), 'same', (1, 1)), (11, 11, 6, 3, 2, 10, (2, 3), 'same', (2, 1))])
def test_conv_ebops_closed_form_is_exact(dev, case):
    """hgq_conv2d_ebops against the definition it replaces (sum of the convolution of the bit-width
    tensors, src/hgq/layers/conv.py:91-102), in integer arithmetic, and its gradients via autograd."""
    from hgq2_amd import ops

    H, W, C, kh, kw, Fo, strides, padding, dilation = case
    g = torch.Generator().manual_seed(H * W)
    bi = torch.randint(0, 13, (1, H, W, C), generator=g).float()
    bk = torch.randint(0, 9, (kh, kw, C, Fo), generator=g).float()
    bir, bkr = bi.clone().requires_grad_(True), bk.clone().requires_grad_(True)
    want = _ref_conv(bir.double(), bkr.double(), None, strides, padding, dilation, False).sum()
    want.backward()
    bip, bkp = bi.to(dev).requires_grad_(True), bk.to(dev).requires_grad_(True)
    got = ops.conv2d_ebops(bip, bkp, strides, padding, dilation)
    (got * 3.0).backward()
    # the total is one fp32 number: exact below 2**24, correctly rounded partial sums above
    assert abs(float(got) - float(want)) <= (0 if float(want) < 2**24 else 1e-6 * float(want))
    assert torch.equal(bip.grad.cpu().double(), 3.0 * bir.grad.double())
    assert torch.equal(bkp.grad.cpu().double(), 3.0 * bkr.grad.double())


@pytest.mark.parametrize('case', [(12, 10, 3, (3, 3), 6, (1, 1), 'valid', 'SAT'), (9, 9, 4, (3, 2), 5, (2, 1), 'same', 'WRAP'),
                                  (8, 11, 2, (2, 3), 4, (2, 3), 'same', 'SAT_SYM')])
def test_one_launch_conv_ebops_term_equals_the_composed_path(dev, case):
    """The loss term ebops * beta of a QConv2D from the raw quantizer variables in one launch (``hgq_conv2d_ebops_q``)
    against the same layer's generic path (bit-width views, closed-form convolution sum, library algebra for the bias
    term and the factors, autograd): value, uint32 variable, and the gradient of every bit-width variable."""
    from hgq2_amd.config import QuantizerConfig
    from hgq2_amd.layers import QConv2D
    from hgq2_amd.layers.core.base import QLayerBase
    from tests.test_gpu_more_layers import _perturb, readme_scopes

    H, W, C, ksize, Fo, strides, padding, iq_over = case
    g = torch.Generator().manual_seed(H * W + C)
    with readme_scopes(beta0=3e-4):
        layer = QConv2D(Fo, ksize, strides=strides, padding=padding, parallelization_factor=3,
                        iq_conf=QuantizerConfig('kif', 'datalane', overflow_mode=iq_over))
    layer.ebops_factor = 1.5
    x = torch.randn(4, H, W, C, generator=g).to(dev)
    layer(x, training=True)
    _perturb(layer, g)
    with torch.no_grad():  # closed straight-through gates and empty words among the entries
        layer.iq.quantizer._f.view(-1)[::5] = -9.0
        layer.kq.quantizer._b.view(-1)[::7] = 0.0
    variables = [layer.iq.quantizer._f, layer.kq.quantizer._b, layer.bq.quantizer._b]
    if layer.iq.quantizer._i.requires_grad:
        variables.append(layer.iq.quantizer._i)
    shape = (1, H, W, C)
    results = []
    for fused in (True, False):
        for v in variables:
            v.grad = None
        term = layer._ebops_loss_term(shape) if fused else QLayerBase._ebops_loss_term(layer, shape)
        (term * 2.0).backward()
        results.append((float(term), int(layer._ebops.cpu().view(torch.int32)), [v.grad.clone() for v in variables]))
    (t1, e1, g1), (t0, e0, g0) = results
    assert e1 == e0 and e0 > 0
    assert abs(t1 - t0) <= 1e-6 * abs(t0)
    for a, b, v in zip(g1, g0, variables):
        assert torch.allclose(a, b, rtol=1e-6, atol=1e-12), float((a - b).abs().max())


@pytest.mark.parametrize('case', [CASES[0], CASES[1], CASES[4], CASES[7], CASES[9], CASES[10], CASES[15]])
def test_conv2d_backward_slices_sum_to_the_reduced_gradient(dev, case):
    """`hgq_conv2d_bwd_slices` leaves what `hgq_conv2d_bwd` adds up: same data gradient, and the slices, added in slice
    order as the joint reduction adds them, are its kernel and bias gradient."""
    from hgq2_amd import _lib, ops

    B, H, W, C, kh, kw, Fo, strides, padding, dilation, relu, bias = case
    g = torch.Generator().manual_seed(100 + CASES.index(case))
    x = torch.randn(B, H, W, C, generator=g).to(dev)
    w = (torch.randn(kh, kw, C, Fo, generator=g) * 0.3).to(dev)
    b = torch.randn(Fo, generator=g).to(dev) if bias else x.new_empty(0)
    act = _lib.ACT_RELU if relu else _lib.ACT_NONE
    geom = ops.conv_geometry(tuple(x.shape), tuple(w.shape), strides, padding, dilation)
    y = ops.conv2d_fwd(x, w, b, list(geom), act)
    dy = torch.randn(y.shape, generator=g).to(dev) if y.numel() else torch.empty_like(y)
    dx, dqw, dqb = ops.conv2d_bwd(dy, y, x, w, list(geom), act, True, bias)
    dx2, slices = ops.conv2d_bwd_slices(dy, y, x, w, list(geom), act, True)
    assert torch.equal(dx, dx2)
    assert slices.shape[1] == w.numel() + Fo
    outs = [torch.empty(w.numel(), device=dev), torch.empty(Fo, device=dev), x.new_empty(0)]
    ops.reduce_slices_multi_op([slices], outs, [False, False, True])
    assert torch.equal(outs[0].view(w.shape), dqw)
    if bias:
        assert torch.equal(outs[1], dqb)


@pytest.mark.parametrize('shape', [
    # B, H, W, C, k, F, padding, relu, bias, quantized (ties inside the windows)
    (3, 28, 28, 1, 3, 32, 'valid', True, True, False),   # the image configuration's first layer
    (2, 13, 17, 3, 3, 8, 'valid', False, True, True),    # odd output sizes: a trailing row and column without a window
    (2, 12, 40, 1, 5, 16, 'same', True, False, True),    # 5 x 5 'same' keeps the tiles on window boundaries
    (1, 9, 70, 4, 3, 4, 'valid', True, True, False),     # several tiles across
])
def test_convolution_backward_from_the_pooled_gradient(dev, shape):
    """`hgq_conv2d_maxpool_bwd` (the convolution and the 2 x 2 maximum pooling behind it as one autograd node) gives the
    bits of the two nodes one after the other: the same pooled output, data / kernel / bias gradient."""
    from hgq2_amd import _lib, ops

    B, H, W, C, k, Fo, padding, relu, bias, quantized = shape
    g = torch.Generator().manual_seed(B * H + W + Fo)
    x = torch.randn(B, H, W, C, generator=g)
    w = torch.randn(k, k, C, Fo, generator=g) * 0.3
    b = torch.randn(Fo, generator=g) if bias else None
    if quantized:  # few distinct values: equal maxima inside a window
        x, w = torch.round(x * 2) / 2, torch.round(w * 4) / 4
        b = torch.round(b) if bias else None
    act = _lib.ACT_RELU if relu else _lib.ACT_NONE
    geom = ops.conv_geometry((B, H, W, C), (k, k, C, Fo), (1, 1), padding, (1, 1))
    assert ops.conv2d_maxpool_supported(geom, Fo)
    got = []
    for fused in (False, True):
        xs, ws = x.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
        bs = b.to(dev).requires_grad_(True) if bias else None
        if fused:
            yp = ops.conv2d(xs, ws, bs, (1, 1), padding, (1, 1), act, maxpool2=True)
        else:
            yp = ops.pool2d(ops.conv2d(xs, ws, bs, (1, 1), padding, (1, 1), act), (2, 2), (2, 2), 'valid', 'max')
        dyp = torch.randn(yp.shape, generator=torch.Generator().manual_seed(5)).to(dev)
        yp.backward(dyp)
        got.append((yp.detach(), xs.grad, ws.grad, bs.grad if bias else None))
    # pooled output and data gradient bit for bit; the kernel / bias gradient walks the pooling windows instead of the pixels
    # (the same non-zero terms in another order): equal to 1e-5 of the largest entry
    for name, a, f in zip(('pooled output', 'dx', 'dw', 'db'), got[0], got[1]):
        if a is None:
            continue
        if name in ('dw', 'db'):
            assert float((a - f).abs().max()) <= 1e-5 * float(a.abs().max()) + 1e-30, f'{name}: {float((a - f).abs().max())}'
        else:
            assert torch.equal(a, f), f'{name}: {float((a - f).abs().max())}'
    # the entry points that keep the unpooled output (the node above saves a byte per window and filter instead) give the same bits
    xs, ws = x.to(dev), w.to(dev)
    bs = b.to(dev) if bias else xs.new_empty(0)
    y, yp = ops.conv2d_maxpool_fwd(xs, ws, bs, list(geom), act)
    assert torch.equal(yp, got[1][0])
    assert torch.equal(y, ops.conv2d(xs, ws, bs if bias else None, (1, 1), padding, (1, 1), act))
    dyp = torch.randn(yp.shape, generator=torch.Generator().manual_seed(5)).to(dev)
    dx, flat = ops.conv2d_maxpool_bwd(dyp, y, xs, ws, list(geom), act, True, True)
    assert torch.equal(dx, got[1][1]) and torch.equal(flat[:w.numel()].view(w.shape), got[1][2])
    if bias:
        assert torch.equal(flat[w.numel():], got[1][3])
    # and against torch's own kernels in fp64 on the CPU
    xd, wd = x.double().requires_grad_(True), w.double().requires_grad_(True)
    pad = (k - 1) // 2 if padding == 'same' else 0
    yd = torch.nn.functional.conv2d(xd.permute(0, 3, 1, 2), wd.permute(3, 2, 0, 1), b.double() if bias else None, padding=pad)
    ypd = torch.nn.functional.max_pool2d(torch.relu(yd) if relu else yd, 2).permute(0, 2, 3, 1)
    assert float((got[1][0].cpu().double() - ypd.detach()).abs().max()) <= 1e-5 * float(ypd.detach().abs().max())
    if not quantized:  # with ties torch may pick another of the equal maxima
        ypd.backward(torch.randn(ypd.shape, generator=torch.Generator().manual_seed(5)).double())
        for name, f, r in (('dx', got[1][1], xd.grad), ('dw', got[1][2], wd.grad)):
            assert float((f.cpu().double() - r).abs().max()) <= 1e-5 * float(r.abs().max()) + 1e-6, name


def test_unsupported_shapes_of_the_pooled_backward_are_refused(dev):
    from hgq2_amd import ops

    for geom_args, Fo in ((((2, 12, 12, 1), (3, 3, 1, 8), (1, 1), 'same', (1, 1)), 8),    # 3 x 3 'same': tiles off the windows
                          (((2, 12, 12, 1), (3, 3, 1, 6), (1, 1), 'valid', (1, 1)), 6),   # filters not a multiple of 4
                          (((2, 12, 12, 16), (3, 3, 16, 8), (1, 1), 'valid', (1, 1)), 8),  # many input channels
                          (((2, 12, 12, 1), (3, 3, 1, 8), (2, 2), 'valid', (1, 1)), 8)):   # strided
        geom = ops.conv_geometry(*geom_args)
        assert not ops.conv2d_maxpool_supported(geom, Fo)
    x = torch.randn(2, 12, 12, 1, device=dev)
    w = torch.randn(3, 3, 1, 8, device=dev)
    with pytest.raises(ValueError):
        ops.conv2d(x, w, None, (1, 1), 'same', (1, 1), 0, maxpool2=True)


def test_sequential_takes_the_pooling_into_the_convolution(dev):
    """A QConv2D followed by MaxPooling2D((2, 2)) inside a Sequential runs as one node; outputs and losses equal those of the
    layers called one by one bit for bit, gradients to 1e-5 of the tensor's largest entry (the node's kernel / bias gradient
    adds the same terms window by window instead of pixel by pixel)."""
    import copy

    from hgq2_amd import host, ops
    from hgq2_amd.utils import models

    model = models.conv_stack(filters=8, device=dev)
    x = torch.rand(4, 28, 28, 1, generator=torch.Generator().manual_seed(3)).to(dev)
    labels = torch.tensor([1, 0, 7, 3], device=dev)
    twin = models.conv_stack(filters=8, device=dev)
    model(x, training=False), twin(x, training=False)  # build
    twin.load_state_dict(copy.deepcopy(model.state_dict()))
    assert type(model.layers[1]) is host.MaxPooling2D and model.layers[0].absorbs(model.layers[1], x)

    def by_hand(m, inp):
        for layer in m.layers:
            inp = layer(inp, training=True)
        return inp

    out_a = model(x, training=True)
    out_b = by_hand(twin, x)
    assert torch.equal(out_a, out_b)
    ops.sparse_ce(out_a, labels).backward()
    ops.sparse_ce(out_b, labels).backward()
    for (name, pa), (_, pb) in zip(model.named_parameters(), twin.named_parameters()):
        if pa.grad is not None or pb.grad is not None:
            assert float((pa.grad - pb.grad).abs().max()) <= 1e-5 * float(pb.grad.abs().max()) + 1e-30, name


@pytest.mark.parametrize('rows,K,N,relu,bias', [(1024, 3872, 10, False, True), (7, 1500, 16, True, True), (33, 1024, 1, False, False),
                                               (5, 2049, 3, True, False), (4097, 1100, 5, False, True)])
def test_few_filters_behind_a_long_contraction(dev, rows, K, N, relu, bias):
    """A classifier behind a flattened feature map (few rows, K in the thousands, a handful of outputs) has a kernel of
    its own in `hgq_conv2d_fwd`; values against fp64 within 1e-5 of the sum of the terms' magnitudes, the same bits on
    every run."""
    from hgq2_amd import _lib, ops

    g = torch.Generator().manual_seed(rows + K + N)
    x = torch.randn(rows, K, generator=g)
    w = torch.randn(K, N, generator=g) * 0.1
    b = torch.randn(N, generator=g) if bias else None
    act = _lib.ACT_RELU if relu else _lib.ACT_NONE
    runs = [ops.matmul_bias_act(x.to(dev), w.to(dev), b.to(dev) if bias else None, act) for _ in range(2)]
    assert torch.equal(runs[0], runs[1])
    want = x.double() @ w.double() + (b.double() if bias else 0.0)
    scale = x.double().abs() @ w.double().abs() + (b.double().abs() if bias else 0.0)
    if relu:
        want = torch.relu(want)
    err = ((runs[0].cpu().double() - want).abs() / scale).max()
    assert float(err) <= 1e-5, float(err)
