"""Pins for the layer twins and the stateful quantizer branches of the CPU oracle (``oracle/hgq_ref.py``).

Nothing here repeats a formula of the oracle: every expected value comes from a textbook / library routine the layer
must reduce to when its quantizers are the identity (the check the reference makes with ``q_type='dummy'``, reference
tests/test_dense.py:31-46, tests/test_activation.py:58-74, tests/test_batchnorm.py:43-58), from nested Python loops
over tiny inputs, from Python-int brute force (EBOPs: bit-widths are integers), or from a worked example computed by
hand.  A dropped term, a transposed operand or a wrong axis fails at least one of them.
"""

import itertools
import math
from fractions import Fraction

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import fixed_point as fp
from oracle import hgq_ref as ref


class Tracing:
    """What the reference's calibration pass hands to the layers as ``training``: falsy, but equal to 'tracing'
    (reference src/hgq/utils/minmax_trace.py:24-32)."""

    def __bool__(self):
        return False

    def __eq__(self, other):
        return other == 'tracing'


def dummy():
    return ref.RefQuantizer(ref.RefDummyQuantizer())


def rnd_bits(q, g, lo_i=-2, hi_i=4, lo_f=-1, hi_f=7, lo_b=0, hi_b=9, k=None):
    """Fill a quantizer's bit-width variables with random integers (and random sign bits); returns the quantizer."""
    inner = q.quantizer
    with torch.no_grad():
        inner._i.copy_(torch.randint(lo_i, hi_i, inner._i.shape, generator=g).float())
        if inner.q_type == 'kif':
            inner._f.copy_(torch.randint(lo_f, hi_f, inner._f.shape, generator=g).float())
        else:
            inner._b.copy_(torch.randint(lo_b, hi_b, inner._b.shape, generator=g).float())
        if k is None:
            inner._k.copy_(torch.randint(0, 2, inner._k.shape, generator=g).to(torch.uint8))
        else:
            inner._k.fill_(k)
    return q


def int_bits(q, shape):
    """``bits`` of a quantizer as nested Python ints over ``shape``, computed from the raw variables with Python
    arithmetic: KIF max(0, i+f), KBI b; plus the sign bit only for overflow mode SAT
    (reference fixed_point_quantizer.py:92-97, :256-265, :435-449)."""
    inner = q.quantizer
    k = np.broadcast_to(inner._k.numpy().astype(np.int64), shape)
    i = np.broadcast_to(np.rint(inner._i.detach().numpy()).astype(np.int64), shape)
    if inner.q_type == 'kif':
        f = np.broadcast_to(np.rint(inner._f.detach().numpy()).astype(np.int64), shape)
        b = np.maximum(i + f, 0)
    else:
        b = np.broadcast_to(np.rint(inner._b.detach().numpy()).astype(np.int64), shape)
    if inner.overflow_mode == 'SAT':
        b = b + k
    return b.tolist()


# --------------------------------------------------------------------------------------------------------------
# dummy-quantizer reductions
# --------------------------------------------------------------------------------------------------------------
def _dummy_softmax(axes, scaler=1.0):
    exp = ref.RefQUnaryFunctionLUT(lambda x: torch.exp(-x * scaler), dummy(), dummy(), enable_ebops=False)
    inv = ref.RefQUnaryFunctionLUT(lambda x: 1.0 / (x + ref.EPSILON), dummy(), dummy(), enable_ebops=False)
    return ref.RefQSoftmax(axes, exp, inv, dummy(), iq=None, input_scaler=scaler, enable_ebops=False)


@pytest.mark.parametrize('axes', [(-1,), (1,), (1, 2)])
@pytest.mark.parametrize('scaler', [1.0, 0.25])
def test_dummy_qsoftmax_is_softmax(axes, scaler):
    """Reference tests/test_activation.py:58-74: QSoftmax with dummy quantizers equals softmax (atol 1e-6)."""
    g = torch.Generator().manual_seed(11)
    x = torch.randn(7, 5, 6, generator=g) * 3
    axes_n = tuple(a % 3 for a in axes)
    sm = _dummy_softmax(axes_n, scaler)
    got = sm(x, training=False)
    xs = (x.double() * scaler)
    if len(axes_n) == 1:
        want = torch.softmax(xs, dim=axes_n[0])
    else:  # softmax over two axes = softmax over the flattened pair
        want = torch.softmax(xs.reshape(7, 30), dim=1).reshape(7, 5, 6)
    assert torch.allclose(got.double(), want, atol=1e-6), float((got.double() - want).abs().max())
    assert torch.allclose(got.sum(dim=axes_n), torch.ones(()), atol=1e-5)


def test_dummy_qsoftmax_mask_is_softmax_over_kept_entries():
    g = torch.Generator().manual_seed(12)
    x = torch.randn(4, 3, 8, generator=g) * 2
    mask = torch.rand(4, 3, 8, generator=g) > 0.4
    mask[..., 0] = True  # every row keeps at least one entry
    got = _dummy_softmax((2,))(x, training=True, mask=mask)
    want = torch.softmax(torch.where(mask, x.double(), torch.tensor(-math.inf, dtype=torch.float64)), dim=2)
    assert torch.all(got[~mask] == 0)
    assert torch.allclose(got.double(), want, atol=1e-6)


def test_dummy_qmha_is_textbook_attention():
    """QMultiHeadAttention with identity quantizers is softmax(Q K^T / sqrt(d)) V between four affine projections
    (reference src/hgq/layers/attn/mha.py:434-537; the 1/sqrt(d) lives in the softmax's input scaler, :77,339)."""
    g = torch.Generator().manual_seed(13)
    B, T, D, N, H = 3, 6, 10, 2, 4
    x = torch.randn(B, T, D, generator=g)
    W = {n: torch.randn(D, N, H, generator=g) * 0.4 for n in 'qkv'}
    b = {'q': torch.randn(N, H, generator=g), 'k': None, 'v': torch.randn(N, H, generator=g)}
    Wo, bo = torch.randn(N, H, D, generator=g) * 0.4, torch.randn(D, generator=g)

    def proj(n):
        return ref.RefQEinsumDense('abc,cde->abde', W[n], b[n], dummy(), dummy(), dummy() if b[n] is not None else None,
                                   (B, T, D), (T, N, H), enable_ebops=False, oq=dummy())

    od = ref.RefQEinsumDense('abcd,cde->abe', Wo, bo, dummy(), dummy(), dummy(), (B, T, N, H), (T, D), enable_ebops=False)
    mha = ref.RefQMultiHeadAttention(proj('q'), proj('k'), proj('v'), od, _dummy_softmax((3,), 1.0 / math.sqrt(H)), enable_ebops=False)
    got = mha(x, training=False)

    xd = x.double()
    heads = []
    for n in range(N):  # one head at a time, plain matrix products
        q = xd @ W['q'][:, n].double() + b['q'][n].double()
        k = xd @ W['k'][:, n].double()
        v = xd @ W['v'][:, n].double() + b['v'][n].double()
        heads.append(F.scaled_dot_product_attention(q, k, v))  # library routine: softmax(q k^T / sqrt(H)) v
    want = sum(heads[n] @ Wo[n].double() for n in range(N)) + bo.double()
    assert torch.allclose(got.double(), want, atol=2e-5), float((got.double() - want).abs().max())

    # a key mask removes those keys for every query
    keep = torch.ones(B, T, T, dtype=torch.bool)
    keep[:, :, -2:] = False
    got_m = mha(x, training=False, mask=keep)
    heads = []
    for n in range(N):
        q = xd @ W['q'][:, n].double() + b['q'][n].double()
        k = xd @ W['k'][:, n].double()
        v = xd @ W['v'][:, n].double() + b['v'][n].double()
        heads.append(F.scaled_dot_product_attention(q[:, :, :], k[:, :-2], v[:, :-2]))
    want_m = sum(heads[n] @ Wo[n].double() for n in range(N)) + bo.double()
    assert torch.allclose(got_m.double(), want_m, atol=2e-5)


def test_dummy_qmha_with_two_sequence_axes_and_separate_inputs_is_textbook_attention():
    """Inputs [batch, T1, T2, features] (the shapes of reference tests/test_mha.py:31-33: query, value and key with
    different feature sizes): with identity quantizers the layer attends over both sequence axes jointly, i.e. it is
    textbook attention on the flattened sequences.  A wrong letter in either einsum string changes the result."""
    g = torch.Generator().manual_seed(17)
    B, q_seq, k_seq, N, H, Hv = 3, (2, 4), (3, 2), 2, 4, 5
    Dq, Dv, Dk = 8, 9, 10
    xq = torch.randn(B, *q_seq, Dq, generator=g)
    xv = torch.randn(B, *k_seq, Dv, generator=g)
    xk = torch.randn(B, *k_seq, Dk, generator=g)
    Wq, Wk, Wv = (torch.randn(d, N, h, generator=g) * 0.4 for d, h in ((Dq, H), (Dk, H), (Dv, Hv)))
    bq, bv = torch.randn(N, H, generator=g), torch.randn(N, Hv, generator=g)
    Wo, bo = torch.randn(N, Hv, Dq, generator=g) * 0.4, torch.randn(Dq, generator=g)

    def proj(W, b, shape, seq, h):
        return ref.RefQEinsumDense('abcd,def->abcef', W, b, dummy(), dummy(), dummy() if b is not None else None,
                                   shape, seq + (N, h), enable_ebops=False, oq=dummy())

    od = ref.RefQEinsumDense('abcde,def->abcf', Wo, bo, dummy(), dummy(), dummy(), (B,) + q_seq + (N, Hv), q_seq + (Dq,),
                             enable_ebops=False)
    mha = ref.RefQMultiHeadAttention(proj(Wq, bq, tuple(xq.shape), q_seq, H), proj(Wk, None, tuple(xk.shape), k_seq, H),
                                     proj(Wv, bv, tuple(xv.shape), k_seq, Hv), od, _dummy_softmax((4, 5), 1.0 / math.sqrt(H)),
                                     enable_ebops=False)
    got = mha(xq, xv, xk, training=False)
    assert tuple(got.shape) == (B,) + q_seq + (Dq,)

    fq, fv, fk = (t.double().flatten(1, 2) for t in (xq, xv, xk))
    heads = []
    for n in range(N):
        q = fq @ Wq[:, n].double() + bq[n].double()
        k = fk @ Wk[:, n].double()
        v = fv @ Wv[:, n].double() + bv[n].double()
        heads.append(F.scaled_dot_product_attention(q, k, v))
    want = (sum(heads[n] @ Wo[n].double() for n in range(N)) + bo.double()).view(B, *q_seq, Dq)
    assert torch.allclose(got.double(), want, atol=2e-5), float((got.double() - want).abs().max())

    # a mask [batch, T1, T2, S1, S2] is broadcast over the heads
    keep = torch.rand(B, *q_seq, *k_seq, generator=g) > 0.3
    keep[..., 0, 0] = True
    got_m = mha(xq, xv, xk, training=False, mask=keep)
    heads = []
    for n in range(N):
        q = fq @ Wq[:, n].double() + bq[n].double()
        k = fk @ Wk[:, n].double()
        v = fv @ Wv[:, n].double() + bv[n].double()
        heads.append(F.scaled_dot_product_attention(q, k, v, attn_mask=keep.flatten(3, 4).flatten(1, 2)))
    want_m = (sum(heads[n] @ Wo[n].double() for n in range(N)) + bo.double()).view(B, *q_seq, Dq)
    assert torch.allclose(got_m.double(), want_m, atol=2e-5)


def test_attention_equation_strings_of_the_product_and_the_oracle_agree():
    from hgq2_amd.layers.attn._equations import attention_equations, proj_equation

    assert proj_equation(2, 1, 2) == ('abc,cde->abde', 'de', 4)  # the strings Keras documents for rank-3 inputs
    assert proj_equation(2, 2, 1) == ('abcd,cde->abe', 'e', 3)
    for rank in (4, 5, 6):
        axes = tuple(range(1, rank - 2))
        assert attention_equations(rank, axes)[:2] == ref.keras_attention_equations(rank, axes)
    assert ref.keras_attention_equations(4, (1,)) == ('aecd,abcd->acbe', 'acbe,aecd->abcd')


def _same_pads(n, k, s):
    """TensorFlow / Keras 'same': ceil(n/s) outputs, the window grid centred with the odd pixel of padding at the end."""
    out = -(-n // s)
    total = max((out - 1) * s + k - n, 0)
    return out, total // 2


def _loop_conv(x, w, strides, padding):
    """Cross-correlation by nested loops, channels-last input [B,H,W,C], kernel [kh,kw,C,F]."""
    B, H, Wd, C = x.shape
    kh, kw, _, Fo = w.shape
    if padding == 'same':
        oh, ph = _same_pads(H, kh, strides[0])
        ow, pw = _same_pads(Wd, kw, strides[1])
    else:
        oh, ph = (H - kh) // strides[0] + 1, 0
        ow, pw = (Wd - kw) // strides[1] + 1, 0
    out = np.zeros((B, oh, ow, Fo))
    for b_, oy, ox, fo in itertools.product(range(B), range(oh), range(ow), range(Fo)):
        acc = 0.0
        for ky, kx, c in itertools.product(range(kh), range(kw), range(C)):
            iy, ix = oy * strides[0] - ph + ky, ox * strides[1] - pw + kx
            if 0 <= iy < H and 0 <= ix < Wd:
                acc += float(x[b_, iy, ix, c]) * float(w[ky, kx, c, fo])
        out[b_, oy, ox, fo] = acc
    return out


@pytest.mark.parametrize('ksize', [(1, 1), (3, 3), (3, 2), (2, 3)])
@pytest.mark.parametrize('strides', [(1, 1), (2, 1), (2, 3)])
@pytest.mark.parametrize('padding', ['valid', 'same'])
def test_dummy_qconv2d_is_loop_convolution(ksize, strides, padding):
    """Shapes of the reference's convolution tests (tests/test_conv.py:61-95): 6x6x2 images."""
    g = torch.Generator().manual_seed(14)
    x = torch.randn(2, 6, 6, 2, generator=g)
    w = torch.randn(*ksize, 2, 3, generator=g)
    bias = torch.randn(3, generator=g)
    layer = ref.RefQConv2D(w, bias, dummy(), dummy(), dummy(), strides=strides, padding=padding, activation='relu',
                           enable_ebops=False)
    got = layer(x, training=False)
    want = np.maximum(_loop_conv(x.numpy(), w.numpy(), strides, padding) + bias.numpy().astype(np.float64), 0)
    assert tuple(got.shape) == want.shape
    np.testing.assert_allclose(got.detach().numpy(), want, atol=2e-5)


def test_same_padding_identity_kernel_keeps_the_image():
    """An odd kernel with a single 1 at its centre must reproduce the image under 'same' (the window is centred)."""
    g = torch.Generator().manual_seed(15)
    x = torch.randn(1, 5, 7, 1, generator=g)
    w = torch.zeros(3, 5, 1, 1)
    w[1, 2, 0, 0] = 1.0
    layer = ref.RefQConv2D(w, None, dummy(), dummy(), None, padding='same', enable_ebops=False)
    assert torch.equal(layer(x, training=False), x)


@pytest.mark.parametrize('mode', ['max', 'avg'])
@pytest.mark.parametrize('pool,strides', [((2, 2), (2, 2)), ((3, 2), (2, 1)), ((2, 3), (1, 2))])
@pytest.mark.parametrize('padding', ['valid', 'same'])
def test_dummy_qpooling_is_loop_pooling(mode, pool, strides, padding):
    """Windows by nested loops; padded cells never win a maximum and are not counted in a mean (the rule the
    reference's exporter restates, src/hgq/_dais_tracer/layers/pool.py:83-103)."""
    g = torch.Generator().manual_seed(16)
    x = torch.randn(2, 7, 6, 3, generator=g)
    layer = ref.RefQPooling2D(mode, pool, strides, padding, dummy(), enable_ebops=False)
    got = layer(x, training=False).detach().numpy()
    B, H, Wd, C = x.shape
    if padding == 'same':
        oh, ph = _same_pads(H, pool[0], strides[0])
        ow, pw = _same_pads(Wd, pool[1], strides[1])
    else:
        oh, ph, ow, pw = (H - pool[0]) // strides[0] + 1, 0, (Wd - pool[1]) // strides[1] + 1, 0
    want = np.zeros((B, oh, ow, C))
    xn = x.numpy().astype(np.float64)
    for b_, oy, ox, c in itertools.product(range(B), range(oh), range(ow), range(C)):
        cells = [xn[b_, iy, ix, c]
                 for iy in range(oy * strides[0] - ph, oy * strides[0] - ph + pool[0])
                 for ix in range(ox * strides[1] - pw, ox * strides[1] - pw + pool[1])
                 if 0 <= iy < H and 0 <= ix < Wd]
        want[b_, oy, ox, c] = max(cells) if mode == 'max' else sum(cells) / len(cells)
    assert got.shape == want.shape
    np.testing.assert_allclose(got, want, atol=1e-6)


@pytest.mark.parametrize('equation,xshape,wshape,bshape', [
    ('bpf,fh->bph', (5, 4, 3), (3, 6), (6,)),
    ('Bij,ijk->Bik', (5, 4, 3), (4, 3, 2), (4, 2)),       # reference tests/test_dense.py:56-82
    ('abc,cde->abde', (3, 4, 5), (5, 2, 3), (2, 3)),      # attention projection
])
def test_dummy_qeinsum_dense_is_loop_contraction(equation, xshape, wshape, bshape):
    g = torch.Generator().manual_seed(17)
    x, w, b = torch.randn(*xshape, generator=g), torch.randn(*wshape, generator=g), torch.randn(*bshape, generator=g)
    out_tail = torch.einsum(equation, x, w).shape[1:]
    layer = ref.RefQEinsumDense(equation, w, b, dummy(), dummy(), dummy(), xshape, tuple(out_tail), activation='relu', enable_ebops=False)
    got = layer(x, training=False)
    # index-by-index contraction written from the equation's letters
    ins, out = equation.split('->')
    a_, b_ = ins.split(',')
    sizes = {}
    for letters, t in ((a_, x), (b_, w)):
        for ch, n in zip(letters, t.shape):
            sizes[ch] = n
    letters = sorted(sizes)
    want = np.zeros([sizes[c] for c in out])
    for idx in itertools.product(*(range(sizes[c]) for c in letters)):
        at = dict(zip(letters, idx))
        want[tuple(at[c] for c in out)] += float(x[tuple(at[c] for c in a_)]) * float(w[tuple(at[c] for c in b_)])
    want = np.maximum(want + b.numpy().astype(np.float64), 0)
    np.testing.assert_allclose(got.detach().numpy(), want, atol=2e-5)


@pytest.mark.parametrize('training', [True, False])
def test_dummy_qeinsum_dense_batchnorm_is_batchnorm_of_the_contraction(training):
    """Folding identity (reference src/hgq/layers/einsum_dense_batchnorm.py:158-211): with identity quantizers the
    layer is gamma * (z - mean) / sqrt(var + eps) + bias with z = einsum(x, W) WITHOUT the bias, batch moments when
    training, moving moments otherwise; eps is the global 1e-7."""
    g = torch.Generator().manual_seed(18)
    x = torch.randn(9, 4, 5, generator=g)
    w = torch.randn(5, 6, generator=g)
    b, gamma = torch.randn(6, generator=g), torch.rand(6, generator=g) + 0.5
    mm, mv = torch.randn(6, generator=g), torch.rand(6, generator=g) + 0.3
    layer = ref.RefQEinsumDenseBatchnorm('bpf,fh->bph', w, b, dummy(), dummy(), dummy(), (9, 4, 5), (4, 6), enable_ebops=False,
                                         gamma=gamma, moving_mean=mm, moving_variance=mv, normalize_axes='h', momentum=0.9)
    got = layer(x, training=training)
    z = torch.einsum('bpf,fh->bph', x.double(), w.double())
    if training:
        mean = z.mean(dim=(0, 1))
        var = ((z - mean) ** 2).mean(dim=(0, 1))
        # library routine: batch normalisation of z with beta = the layer's bias
        want = F.batch_norm(z.reshape(-1, 6), None, None, gamma.double(), b.double(), True, 0.0, 1e-7).reshape(z.shape)
        assert torch.allclose(layer.moving_mean.double(), 0.9 * mm.double() + 0.1 * mean, atol=1e-6)
        assert torch.allclose(layer.moving_variance.double(), 0.9 * mv.double() + 0.1 * var, atol=1e-5)
    else:
        want = F.batch_norm(z.reshape(-1, 6), mm.double(), mv.double(), gamma.double(), b.double(), False, 0.0, 1e-7).reshape(z.shape)
        assert torch.equal(layer.moving_mean, mm) and torch.equal(layer.moving_variance, mv)
    assert torch.allclose(got.double(), want, atol=3e-5), float((got.double() - want).abs().max())


def test_qeinsum_dense_batchnorm_gradient_flows_through_the_batch_moments():
    """The batch moments are part of the graph when training: d/dW of sum(y * r) must equal that of the batch-norm
    library routine (which differentiates through its own statistics)."""
    g = torch.Generator().manual_seed(19)
    x = torch.randn(12, 3, 4, generator=g)
    w = torch.randn(4, 5, generator=g)
    b, gamma = torch.randn(5, generator=g), torch.rand(5, generator=g) + 0.5
    r = torch.randn(12, 3, 5, generator=g)
    layer = ref.RefQEinsumDenseBatchnorm('bpf,fh->bph', w, b, dummy(), dummy(), dummy(), (12, 3, 4), (3, 5), enable_ebops=False,
                                         gamma=gamma, moving_mean=torch.zeros(5), moving_variance=torch.ones(5), normalize_axes='h')
    (layer(x, training=True) * r).sum().backward()
    wd = w.double().requires_grad_(True)
    gd = gamma.double().requires_grad_(True)
    z = torch.einsum('bpf,fh->bph', x.double(), wd)
    y = F.batch_norm(z.reshape(-1, 5), None, None, gd, b.double(), True, 0.0, 1e-7).reshape(z.shape)
    (y * r.double()).sum().backward()
    assert torch.allclose(layer.kernel.grad.double(), wd.grad, atol=1e-4, rtol=1e-4)
    assert torch.allclose(layer.gamma.grad.double(), gd.grad, atol=1e-4, rtol=1e-4)


# --------------------------------------------------------------------------------------------------------------
# EBOPs: Python-int brute force
# --------------------------------------------------------------------------------------------------------------
def _q(place, shape, q_type, overflow, g, k=None, **kw):
    return rnd_bits(ref.default_quantizer(place, shape, q_type=q_type, overflow_mode=overflow, **kw), g, k=k)


@pytest.mark.parametrize('iq_over', ['WRAP', 'SAT'])
def test_ebops_einsum_dense_bruteforce(iq_over):
    """Reference src/hgq/layers/core/einsum_dense.py:85-93 with n_parallel from :10-20."""
    g = torch.Generator().manual_seed(21)
    P, Fi, H = 3, 4, 5
    iq = _q('datalane', (None, P, Fi), 'kif', iq_over, g)
    kq = _q('weight', (Fi, H), 'kbi', 'SAT_SYM', g)
    bq = _q('bias', (H,), 'kbi', 'SAT', g)
    for pf in (-1, 2):
        layer = ref.RefQEinsumDense('bpf,fh->bph', torch.zeros(Fi, H), torch.zeros(H), iq, kq, bq, (7, P, Fi), (P, H),
                                    parallelization_factor=pf)
        bi, bk, bb = int_bits(iq, (1, P, Fi)), int_bits(kq, (Fi, H)), int_bits(bq, (H,))
        mac = sum(bi[0][p][f] * bk[f][h] for p in range(P) for f in range(Fi) for h in range(H))
        want = (mac + Fraction(sum(bb), H) * (P * H)) * (pf if pf > 0 else P) / P   # n_parallel = P (free axis of the input)
        assert float(layer._compute_ebops((1, P, Fi))) == pytest.approx(float(want), rel=1e-6)


def test_einsum_free0_size():
    """Reference src/hgq/layers/core/einsum_dense.py:10-20: product of the input's non-batch axes that are not
    contracted and not shared with the kernel."""
    assert ref._einsum_free0_size('bpf,fh->bph', (None, 64, 16)) == 64
    assert ref._einsum_free0_size('abc,cde->abde', (None, 7, 5)) == 7
    assert ref._einsum_free0_size('Bij,ijk->Bik', (None, 4, 3)) == 1     # i is shared with the kernel
    assert ref._einsum_free0_size('abcd,cde->abe', (None, 6, 2, 4)) == 6


@pytest.mark.parametrize('padding,strides', [('valid', (1, 1)), ('same', (1, 1)), ('valid', (2, 1)), ('same', (2, 2))])
def test_ebops_conv2d_bruteforce(padding, strides):
    """Reference src/hgq/layers/conv.py:91-102: the sum over every output pixel and filter of bits_in * bits_ker under
    the window, by nested loops over Python ints; parallelization factor scales the contraction part only."""
    g = torch.Generator().manual_seed(22)
    Hh, Ww, C, Fo, kh, kw = 5, 4, 2, 3, 3, 2
    iq = _q('datalane', (None, Hh, Ww, C), 'kif', 'WRAP', g)
    kq = _q('weight', (kh, kw, C, Fo), 'kbi', 'SAT_SYM', g)
    bq = _q('bias', (Fo,), 'kbi', 'SAT_SYM', g)
    bi, bk, bb = int_bits(iq, (1, Hh, Ww, C)), int_bits(kq, (kh, kw, C, Fo)), int_bits(bq, (Fo,))
    if padding == 'same':
        oh, ph = _same_pads(Hh, kh, strides[0])
        ow, pw = _same_pads(Ww, kw, strides[1])
    else:
        oh, ph, ow, pw = (Hh - kh) // strides[0] + 1, 0, (Ww - kw) // strides[1] + 1, 0
    mac = 0
    for oy, ox, fo, ky, kx, c in itertools.product(range(oh), range(ow), range(Fo), range(kh), range(kw), range(C)):
        iy, ix = oy * strides[0] - ph + ky, ox * strides[1] - pw + kx
        if 0 <= iy < Hh and 0 <= ix < Ww:
            mac += bi[0][iy][ix][c] * bk[ky][kx][c][fo]
    n_parallel = oh * ow
    for pf in (-1, 1, 3):
        layer = ref.RefQConv2D(torch.zeros(kh, kw, C, Fo), torch.zeros(Fo), iq, kq, bq, strides=strides, padding=padding,
                               parallelization_factor=pf, n_parallel=n_parallel)
        want = Fraction(mac) * (pf if pf > 0 else n_parallel) / n_parallel + Fraction(sum(bb), Fo) * (Hh * Ww * Fo)
        assert float(layer._compute_ebops((1, Hh, Ww, C))) == pytest.approx(float(want), rel=1e-6)


def test_ebops_lut_bruteforce():
    """Reference src/hgq/layers/activation.py:63-67: sum 2**bits_in * bits_out * 1e-4."""
    g = torch.Generator().manual_seed(23)
    shape = (1, 3, 4)
    iq = _q('datalane', (None, 3, 4), 'kif', 'SAT', g)
    oq = _q('table', (None, 3, 4), 'kbi', 'SAT', g, homogeneous_axis=(0,))
    lut = ref.RefQUnaryFunctionLUT(torch.exp, iq, oq)
    bi, bo = int_bits(iq, shape), int_bits(oq, shape)
    want = sum(Fraction(2) ** bi[0][a][b] * bo[0][a][b] for a in range(3) for b in range(4)) / 10000
    assert float(lut._compute_ebops(shape)) == pytest.approx(float(want), rel=1e-6)


@pytest.mark.parametrize('with_iq', [False, True])
@pytest.mark.parametrize('pf', [-1, 2])
def test_ebops_softmax_bruteforce(with_iq, pf):
    """Reference src/hgq/layers/softmax.py:134-161 (stable form): subtract + accumulate + multiply, scaled by
    n_instance / max_instance."""
    g = torch.Generator().manual_seed(24)
    A, S = 3, 4
    shape = (1, A, S)
    exp_iq = _q('datalane', (None, A, S), 'kif', 'SAT', g, heterogeneous_axis=())
    exp_oq = _q('table', (None, A, S), 'kbi', 'SAT', g, homogeneous_axis=(0,), k=0)
    inv_iq = _q('datalane', (None, A, 1), 'kif', 'WRAP', g, heterogeneous_axis=())
    inv_oq = _q('table', (None, A, 1), 'kbi', 'SAT', g, homogeneous_axis=(0,), k=0)
    iq = _q('datalane', (None, A, S), 'kif', 'WRAP', g) if with_iq else None
    exp = ref.RefQUnaryFunctionLUT(None, exp_iq, exp_oq)
    inv = ref.RefQUnaryFunctionLUT(None, inv_iq, inv_oq)
    sm = ref.RefQSoftmax((2,), exp, inv, None, iq=iq, parallelization_factor=pf)
    be, bv = int_bits(exp_oq, shape), int_bits(inv_oq, (1, A, 1))
    bsub = int_bits(iq if with_iq else exp_iq, shape)
    sub = sum(bsub[0][a][s] for a in range(A) for s in range(S))
    accum = sum(sum(be[0][a]) - min(be[0][a]) for a in range(A))
    mult = sum(be[0][a][s] * bv[0][a][0] for a in range(A) for s in range(S))
    want = Fraction(sub + accum + mult) * (pf if pf > 0 else A) / A
    assert float(sm._compute_ebops(shape)) == pytest.approx(float(want), rel=1e-6)


def test_unstable_softmax_form_is_softmax_and_counts_its_exp_table_itself():
    """``stable=False`` (reference src/hgq/layers/softmax.py:49-53,87-96,116-120,150-152): no maximum is subtracted and the
    exp table evaluates exp(+x * scaler) without an input quantizer, so with dummy quantizers the layer is still softmax;
    in the EBOPs the subtraction drops out and the table size sum(2^input bits * exp bits) * 1e-4 is counted here."""
    g = torch.Generator().manual_seed(27)
    x = torch.randn(6, 3, 4, generator=g)
    exp = ref.RefQUnaryFunctionLUT(lambda t: torch.exp(t * 0.5), None, dummy(), enable_ebops=False)
    inv = ref.RefQUnaryFunctionLUT(lambda t: 1.0 / (t + ref.EPSILON), dummy(), dummy(), enable_ebops=False)
    sm = ref.RefQSoftmax((2,), exp, inv, dummy(), iq=None, input_scaler=0.5, enable_ebops=False, stable=False)
    assert torch.allclose(sm(x, training=False).double(), torch.softmax(x.double() * 0.5, dim=2), atol=1e-6)

    A, S = 3, 4
    shape = (1, A, S)
    exp_oq = _q('table', (None, A, S), 'kbi', 'SAT', g, homogeneous_axis=(0,), k=0)
    inv_iq = _q('datalane', (None, A, 1), 'kif', 'WRAP', g, heterogeneous_axis=())
    inv_oq = _q('table', (None, A, 1), 'kbi', 'SAT', g, homogeneous_axis=(0,), k=0)
    iq = _q('datalane', (None, A, S), 'kif', 'WRAP', g)
    sm = ref.RefQSoftmax((2,), ref.RefQUnaryFunctionLUT(None, None, exp_oq, enable_ebops=False), ref.RefQUnaryFunctionLUT(None, inv_iq, inv_oq),
                         None, iq=iq, stable=False)
    be, bv, bi = int_bits(exp_oq, shape), int_bits(inv_oq, (1, A, 1)), int_bits(iq, shape)
    accum = sum(sum(be[0][a]) - min(be[0][a]) for a in range(A))
    mult = sum(be[0][a][s] * bv[0][a][0] for a in range(A) for s in range(S))
    table = sum(Fraction(2) ** bi[0][a][s] * be[0][a][s] for a in range(A) for s in range(S)) / 10000
    assert float(sm._compute_ebops(shape)) == pytest.approx(float(accum + mult + table), rel=1e-6)


def test_ebops_mha_bruteforce():
    """Reference src/hgq/layers/attn/mha.py:386-416: every (query position, key position, head, channel) product of
    the two attention contractions, by nested loops over Python ints."""
    g = torch.Generator().manual_seed(25)
    T, N, H = 3, 2, 4
    oq = {n: _q('datalane', (None, T, N, H), 'kif', 'WRAP', g) for n in 'qkv'}
    soq = _q('datalane', (None, N, T, T), 'kif', 'WRAP', g)
    mk = lambda n: ref.RefQEinsumDense('abc,cde->abde', torch.zeros(5, N, H), None, dummy(), dummy(), None, (2, T, 5), (T, N, H),  # noqa: E731
                                       enable_ebops=False, oq=oq[n])
    sm = ref.RefQSoftmax((3,), ref.RefQUnaryFunctionLUT(None, dummy(), dummy(), enable_ebops=False),
                         ref.RefQUnaryFunctionLUT(None, dummy(), dummy(), enable_ebops=False), soq, enable_ebops=False)
    mha = ref.RefQMultiHeadAttention(mk('q'), mk('k'), mk('v'), None, sm)
    mha._shapes = ((2, T, N, H), (2, T, N, H), (2, T, N, H), (2, N, T, T))
    bq_, bk_, bv_ = (int_bits(oq[n], (1, T, N, H)) for n in 'qkv')
    ba = int_bits(soq, (1, N, T, T))
    qk = sum(bq_[0][t][n][h] * bk_[0][s][n][h] for t in range(T) for s in range(T) for n in range(N) for h in range(H))
    av = sum(ba[0][n][t][s] * bv_[0][s][n][h] for t in range(T) for s in range(T) for n in range(N) for h in range(H))
    assert float(mha._compute_ebops()) == float(qk + av)
    mha.parallelization_factor = 3
    assert float(mha._compute_ebops()) == float(3 * (qk + av))


def test_ebops_mha_two_sequence_axes_bruteforce():
    """The same count for inputs with two sequence axes and different query / key sequence shapes: every
    (query position, key position, head, channel) product, positions being pairs."""
    g = torch.Generator().manual_seed(26)
    (T1, T2), (S1, S2), N, H, Hv = (2, 3), (3, 2), 2, 3, 4
    oq = {'q': _q('datalane', (None, T1, T2, N, H), 'kif', 'WRAP', g), 'k': _q('datalane', (None, S1, S2, N, H), 'kif', 'WRAP', g),
          'v': _q('datalane', (None, S1, S2, N, Hv), 'kif', 'WRAP', g)}
    soq = _q('datalane', (None, N, T1, T2, S1, S2), 'kif', 'WRAP', g)
    sm = ref.RefQSoftmax((4, 5), ref.RefQUnaryFunctionLUT(None, dummy(), dummy(), enable_ebops=False),
                         ref.RefQUnaryFunctionLUT(None, dummy(), dummy(), enable_ebops=False), soq, enable_ebops=False)
    holder = lambda q: type('P', (), {'oq': q})()  # noqa: E731  (only the projections' output quantizers enter)
    mha = ref.RefQMultiHeadAttention(holder(oq['q']), holder(oq['k']), holder(oq['v']), None, sm)
    mha._shapes = ((5, T1, T2, N, H), (5, S1, S2, N, H), (5, S1, S2, N, Hv), (5, N, T1, T2, S1, S2))
    bq_, bk_, bv_ = int_bits(oq['q'], (1, T1, T2, N, H)), int_bits(oq['k'], (1, S1, S2, N, H)), int_bits(oq['v'], (1, S1, S2, N, Hv))
    ba = int_bits(soq, (1, N, T1, T2, S1, S2))
    pos = [(t1, t2, s1, s2) for t1 in range(T1) for t2 in range(T2) for s1 in range(S1) for s2 in range(S2)]
    qk = sum(bq_[0][t1][t2][n][h] * bk_[0][s1][s2][n][h] for t1, t2, s1, s2 in pos for n in range(N) for h in range(H))
    av = sum(ba[0][n][t1][t2][s1][s2] * bv_[0][s1][s2][n][h] for t1, t2, s1, s2 in pos for n in range(N) for h in range(Hv))
    assert float(mha._compute_ebops()) == float(qk + av)


def test_ebops_pooling_and_batchnorm_bruteforce():
    """Reference src/hgq/layers/pooling.py:28-30 (sum of the input bits, scaled) and
    src/hgq/layers/batch_normalization.py (sum bits_in * bits_scale per channel + mean(bits_offset) * size)."""
    g = torch.Generator().manual_seed(26)
    Hh, Ww, C = 4, 3, 2
    iq = _q('datalane', (None, Hh, Ww, C), 'kif', 'WRAP', g)
    bi = int_bits(iq, (1, Hh, Ww, C))
    total = sum(bi[0][y][x][c] for y in range(Hh) for x in range(Ww) for c in range(C))
    pool = ref.RefQPooling2D('max', (2, 2), (2, 2), 'valid', iq, parallelization_factor=1, n_parallel=2)
    assert float(pool._compute_ebops((1, Hh, Ww, C))) == float(Fraction(total, 2))
    kq = _q('weight', (C,), 'kbi', 'SAT_SYM', g)
    bq = _q('bias', (C,), 'kbi', 'SAT_SYM', g)
    bn = ref.RefQBatchNormalization(-1, torch.ones(C), torch.zeros(C), torch.zeros(C), torch.ones(C), iq, kq, bq)
    bk, bb = int_bits(kq, (C,)), int_bits(bq, (C,))
    want = sum(bi[0][y][x][c] * bk[c] for y in range(Hh) for x in range(Ww) for c in range(C)) + Fraction(sum(bb), C) * (Hh * Ww * C)
    assert float(bn._compute_ebops((1, Hh, Ww, C))) == pytest.approx(float(want), rel=1e-6)


def test_call_wrapper_assigns_truncated_ebops_and_beta_term():
    """Reference src/hgq/layers/core/base.py:95-104: ``_ebops`` is the float estimate cast to uint32 (truncation) and
    the loss term is estimate * beta; neither is produced at inference."""
    g = torch.Generator().manual_seed(27)
    iq = _q('datalane', (None, 3, 4), 'kif', 'SAT', g, k=1)
    oq = _q('table', (None, 3, 4), 'kbi', 'SAT', g, homogeneous_axis=(0,), k=0)
    lut = ref.RefQUnaryFunctionLUT(lambda x: x, iq, oq, beta0=0.5)
    x = torch.randn(2, 3, 4, generator=g)
    lut(x, training=False)
    assert lut.losses == [] and int(lut.ebops_value) == 0
    lut(x, training=True)
    est = float(lut._compute_ebops((1, 3, 4)))
    assert est != int(est)  # the 1e-4 factor makes it fractional, so truncation is visible
    assert int(lut.ebops_value) == int(est)
    assert float(lut.losses[0]) == pytest.approx(0.5 * est, rel=1e-6)


# --------------------------------------------------------------------------------------------------------------
# stateful quantizer branches: worked examples
# --------------------------------------------------------------------------------------------------------------
def test_kbi_wrap_training_worked_example():
    """Reference fixed_point_quantizer.py:277-288 + :16-22.  b = 4 per column, batch-shared.  The integer bits come
    from the UN-rounded input: least i with max|x| <= 2**i * (1 - 2**-b) (eps terms aside), then max with the
    decayed state, then the constraint; the variable is assigned first, so the output is round(x, f = b - round(i_new))."""
    q = ref.default_quantizer('datalane', (None, 3), q_type='kbi', overflow_mode='WRAP', ic=('minmax', -2.0, 3.0))
    inner = q.quantizer
    with torch.no_grad():
        inner._b.fill_(4.0)
        inner._i.copy_(torch.tensor([[2.0, 0.0, 1.0]]))
    x = torch.tensor([[0.30, -1.90, 20.0], [-0.45, 1.00, -3.0]])
    y = q(x, training=True)
    # col0: .45/(15/16)=.48 -> i=-1, max(2-.01, -1) = 1.99 ; col1: 1.9/(15/16)=2.03 -> i=2 > -0.01
    # col2: 20/(15/16)=21.3 -> i=5, clipped to 3 by the constraint
    assert torch.allclose(inner._i, torch.tensor([[1.99, 2.0, 3.0]]))
    # f = b - round(i_new) = [2, 2, 1] -> steps .25, .25, .5 ; RND = floor(x/step + .5)*step: -1.9*4 = -7.6 -> -8 -> -2.0
    want = torch.tensor([[0.25, -2.0, 20.0], [-0.5, 1.0, -3.0]])
    assert torch.equal(y, want)
    assert inner._k.tolist() == [[1, 1, 1]]  # training never touches the sign bit


def test_kbi_wrap_tracing_worked_example():
    """Reference fixed_point_quantizer.py:289-300: tracing grows i from the rounded state (no decay), rounds with
    f = b - NEW i, and ORs 'any rounded value negative' (and b > 0) into k."""
    q = ref.default_quantizer('datalane', (None, 4), q_type='kbi', overflow_mode='WRAP')
    inner = q.quantizer
    with torch.no_grad():
        inner._b.copy_(torch.tensor([[4.0, 4.0, 0.0, 4.0]]))
        inner._i.copy_(torch.tensor([[-1e9, 1.4, -1e9, -1e9]]))
        inner._k.zero_()
    x = torch.tensor([[0.30, -0.20, -5.0, -0.01], [0.45, 0.10, 1.0, 0.9]])
    y = q(x, training=Tracing())
    # col0: max .45 -> i=-1, f=5: step 1/32 -> .3125 , .4375(.45*32=14.4 -> 14) ; no negative
    # col1: state round(1.4)=1 beats i(.2)=-2 ; f=3 -> -0.25 (floor(-1.6+.5)=-2) and .125 ; negative seen -> k=1
    # col2: b=0 -> i=32 (sentinel), f=-32 -> everything rounds to 0 ; k stays 0 because b == 0
    # col3: max .9 -> i=0, f=4: -0.01*16=-.16 -> floor(.34)=0 -> 0.0 (no negative AFTER rounding), .9 -> 14/16
    want = torch.tensor([[0.3125, -0.25, 0.0, 0.0], [0.4375, 0.125, 0.0, 0.875]])
    assert torch.equal(y, want)
    assert inner._i.tolist() == [[-1.0, 1.0, 32.0, 0.0]]
    assert inner._k.tolist() == [[0, 1, 0, 0]]


def test_kif_wrap_tracing_worked_example():
    """Reference fixed_point_quantizer.py:414-422: the constraint is applied to the candidate BEFORE the max with the
    rounded state; k collects negatives of the rounded input."""
    q = ref.default_quantizer('datalane', (None, 3), q_type='kif', overflow_mode='WRAP', ic=('minmax', -23.0, 4.0))
    inner = q.quantizer
    with torch.no_grad():
        inner._f.copy_(torch.tensor([[2.0, 2.0, 0.0]]))
        inner._i.copy_(torch.tensor([[-1e9, 2.6, -1e9]]))
        inner._k.zero_()
    x = torch.tensor([[1.80, 0.10, 100.0], [-0.10, 0.30, 3.0]])
    y = q(x, training=Tracing())
    # col0: round(1.8, f=2) = 1.75 ; 1.75 + .25 = 2 -> i = 1 ; -0.10 -> floor(-.4+.5)=0 -> no negative
    # col1: max .25 -> ceil(log2(.5)) = -1 ; state round(2.6) = 3 wins
    # col2: 100 + 1 -> ceil(log2 101) = 7 -> clipped to 4 by the constraint
    assert torch.equal(y, torch.tensor([[1.75, 0.0, 100.0], [0.0, 0.25, 3.0]]))
    assert inner._i.tolist() == [[1.0, 3.0, 4.0]]
    assert inner._k.tolist() == [[0, 0, 0]]
    q(torch.tensor([[-1.0, 0.0, 0.0]]), training=Tracing())
    assert inner._k.tolist() == [[1, 0, 0]] and inner._i.tolist() == [[1.0, 3.0, 4.0]]


def test_kif_wrap_training_ignores_the_constraint():
    """Reference fixed_point_quantizer.py:409-413: in the training branch the constraint lands on a dead value."""
    q = ref.default_quantizer('datalane', (None, 1), q_type='kif', overflow_mode='WRAP', ic=('minmax', -23.0, 3.0))
    q(torch.tensor([[1000.0]]), training=True)
    assert q.quantizer._i.tolist() == [[10.0]]  # ceil(log2(1000 + 2**-6)) = 10 > 3


def test_wrap_inference_wraps_and_zeroes_empty_words():
    """Reference fixed_point_quantizer.py:142-150 for a WRAP quantizer at inference: two's-complement wrap of the
    rounded value, and zero wherever k + i + f <= 0."""
    q = ref.default_quantizer('datalane', (None, 3), q_type='kif', overflow_mode='WRAP')
    inner = q.quantizer
    with torch.no_grad():
        inner._i.copy_(torch.tensor([[1.0, 1.0, -3.0]]))
        inner._f.copy_(torch.tensor([[1.0, 1.0, 2.0]]))
        inner._k.copy_(torch.tensor([[1, 0, 1]], dtype=torch.uint8))
    y = q(torch.tensor([[2.0, 2.0, 0.7], [-2.5, -0.5, -0.7]]), training=False)
    # col0: signed, range [-2, 1.5]: 2.0 -> -2.0 ; -2.5 -> floor(-5+.5)=-5 halves -> +3 halves = 1.5
    # col1: unsigned, range [0, 1.5]: 2.0 -> 0 ; -0.5 -> 1.5
    # col2: k+i+f = 0 -> 0
    assert torch.equal(y, torch.tensor([[-2.0, 0.0, 0.0], [1.5, 1.5, 0.0]]))


def test_weight_quantizer_rnd_wrap_returns_rounded_only():
    """Reference fixed_point_quantizer.py:302-305 / :426-427: a WRAP weight quantizer outside training rounds only."""
    for q_type in ('kif', 'kbi'):
        q = ref.default_quantizer('weight', (2,), q_type=q_type, overflow_mode='WRAP')
        inner = q.quantizer
        with torch.no_grad():
            inner._i.fill_(0.0)
            (inner._f if q_type == 'kif' else inner._b).fill_(2.0)
        y = q(torch.tensor([5.3, -7.6]), training=False)
        assert torch.equal(y, torch.tensor([5.25, -7.5]))  # far outside [-1, .75], yet not wrapped


# --------------------------------------------------------------------------------------------------------------
# Quantizer wrapper, surrogate gradient model
# --------------------------------------------------------------------------------------------------------------
def test_quantizer_wrapper_scaler_qnoise_affine_worked_example():
    """Reference src/hgq/quantizer/quantizer.py:49-60 on a quantizer with step 1 (f = 0), RND:
    x = 5.2, scaler 2 -> 2.6 -> q = 3 -> *2 = 6 ; qnoise 0.5 (training only) blends with the SCALED input:
    2.6 + 0.5 * (6 - 2.6) = 4.3 ; affine (3, -1) -> 11.9 ; at inference: 6 * 3 - 1 = 17."""
    inner = ref.default_quantizer('datalane', (None, 1), q_type='kif', overflow_mode='SAT', f0=0, i0=6).quantizer
    x = torch.tensor([[5.2]])
    full = ref.RefQuantizer(inner, scaler=2.0, affine=(3.0, -1.0), qnoise_factor=0.5)
    assert float(full(x, training=True)) == pytest.approx(11.9, rel=1e-6)
    assert float(full(x, training=False)) == pytest.approx(17.0, rel=1e-6)
    assert float(ref.RefQuantizer(inner, scaler=2.0)(x, training=True)) == 6.0
    assert float(ref.RefQuantizer(inner, qnoise_factor=0.25)(x, training=True)) == pytest.approx(5.2 + 0.25 * (5.0 - 5.2), rel=1e-6)
    assert float(ref.RefQuantizer(inner, affine=(0.5, 1.0))(x, training=False)) == 3.5


def test_rounding_surrogate_is_the_derivative_of_the_stated_error_model():
    """The rounding surrogate's model: the rounding error delta = xq - x scales with the step, delta(f + h) =
    delta(f) * 2**-h, and x is passed straight through.  Differentiating THAT model numerically (central difference
    in float64) must give what the oracle's backward returns for d/df; a wrong sign or a missing ln 2 shows.  Whether
    the third-party package uses this model cannot be checked here (it is not installed)."""
    g = torch.Generator().manual_seed(31)
    x = (torch.randn(256, generator=g) * 3).requires_grad_(True)
    f = torch.randint(0, 6, (256,), generator=g).float().requires_grad_(True)
    for mode in ('RND', 'TRN', 'RND_CONV'):
        x.grad = f.grad = None
        y = fp.fixed_round(x, f, mode, True)
        up = torch.randn(256, generator=g)
        (y * up).sum().backward()
        delta = (y.detach() - x.detach()).double()
        h = 1e-6
        model = lambda hh: x.detach().double() + delta * 2.0 ** (-hh)  # noqa: E731
        want_df = (model(h) - model(-h)) / (2 * h) * up.double()
        assert torch.allclose(f.grad.double(), want_df, rtol=1e-5, atol=1e-9)
        assert torch.equal(x.grad, up)
