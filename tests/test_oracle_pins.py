"""Pins for the CPU oracle: every check here is independent of the oracle's own formulas
(exact integer/rational arithmetic, closed forms stated in the reference, finite
differences, textbook routines)."""

import itertools
import math
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import exact
from oracle import fixed_point as fp
from oracle import hgq_ref as ref

ROUND = ('TRN', 'RND', 'RND_CONV')
OVER = ('WRAP', 'SAT', 'SAT_SYM')


def _grid(i, f):
    """Dense grid with exact ties, both range edges and values far outside the range."""
    step = Fraction(2) ** (-(f + 2))  # quarter-LSB steps -> hits .25 .5 .75 ties exactly
    top = Fraction(2) ** (i + 1) + 3
    n = int(top / step)
    n = min(n, 3000)
    pts = [float(step * j) for j in range(-n, n + 1)]
    edge = Fraction(2) ** i
    for d in (-2, -1, 0, 1, 2):
        pts += [float(edge + d * step), float(-edge + d * step)]
    return np.unique(np.asarray(pts, dtype=np.float32))


@pytest.mark.parametrize('round_mode', ROUND)
@pytest.mark.parametrize('overflow_mode', OVER)
def test_forward_values_match_exact_ap_fixed(round_mode, overflow_mode):
    q = fp.get_fixed_quantizer(round_mode, overflow_mode)
    rng = np.random.default_rng(0)
    n_checked = 0
    for k, i, f in itertools.product((0, 1), range(-4, 7), range(-4, 9)):
        if i + f < 0 or k + i + f <= 0:
            continue
        xs = np.concatenate([_grid(i, f), rng.normal(0, 2.0 ** (i + 0.5), 64).astype(np.float32)])
        x = torch.from_numpy(xs)
        kk, ii, ff = (torch.full_like(x, float(v)) for v in (k, i, f))
        y = q(x, kk, ii, ff, False, None).numpy()
        want = np.array([float(exact.exact_quantize(float(v), k, i, f, round_mode, overflow_mode)) for v in xs], dtype=np.float32)
        np.testing.assert_array_equal(y, want, err_msg=f'k={k} i={i} f={f}')
        n_checked += len(xs)
    assert n_checked > 50_000


@pytest.mark.parametrize('round_mode', ROUND)
@pytest.mark.parametrize('overflow_mode', ('SAT', 'SAT_SYM'))
def test_range_step_idempotence(round_mode, overflow_mode):
    """Closed forms of the reference: fixed_point_quantizer.py:107-120."""
    q = fp.get_fixed_quantizer(round_mode, overflow_mode)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(20000, generator=g) * 8
    k = torch.randint(0, 2, x.shape, generator=g).float()
    i = torch.randint(-2, 5, x.shape, generator=g).float()
    f = torch.randint(-1, 9, x.shape, generator=g).float()
    ok = (k + i + f > 0) & (i + f >= 0)
    x, k, i, f = x[ok], k[ok], i[ok], f[ok]
    y = q(x, k, i, f, True, None)
    hi = 2.0**i - 2.0**-f
    lo = -k * hi if overflow_mode == 'SAT_SYM' else -k * 2.0**i
    assert torch.all(y <= hi) and torch.all(y >= lo)
    assert torch.all(torch.remainder(y, 2.0**-f) == 0)
    assert torch.equal(q(y, k, i, f, True, None), y)


def test_wrap_training_is_round_only():
    """fixed_point_quantizer.py:288,405-424: the WRAP training branch returns round(x, f)."""
    q = fp.get_fixed_quantizer('RND', 'WRAP')
    x = torch.randn(4096) * 30
    f = torch.randint(0, 6, x.shape).float()
    i = torch.zeros_like(x)
    k = torch.ones_like(x)
    y = q(x, k, i, f, True, None)
    assert torch.equal(y, torch.floor(x * 2.0**f + 0.5) / 2.0**f)
    assert torch.equal(y, q.round(x, f, False, None))


def test_minimal_i_given_xf_is_least_sufficient_i():
    rng = np.random.default_rng(3)
    for f in range(-3, 10):
        n = rng.integers(0, 2**12, 200)
        xr = (n * 2.0**-f).astype(np.float32)
        got = ref.minimal_i_given_xf(torch.from_numpy(xr), torch.full((len(xr),), float(f)), symmetric=False).numpy()
        got_sym = ref.minimal_i_given_xf(torch.from_numpy(xr), torch.full((len(xr),), float(f)), symmetric=True).numpy()
        want = np.array([exact.exact_minimal_i_given_xf(float(v), f) for v in xr], dtype=np.float32)
        np.testing.assert_array_equal(got, want)
        np.testing.assert_array_equal(got_sym, want)
        # invariant: value fits with `want` integer bits and not with one less
        assert np.all(xr <= 2.0**want - 2.0**-f)
        assert np.all(xr > 2.0 ** (want - 1) - 2.0**-f)


def test_minimal_i_given_xb_symmetric_invariant():
    """fixed_point_quantizer.py:16-19: least i with x <= 2**i * (1 - 2**-b), up to the eps terms."""
    rng = np.random.default_rng(4)
    for b in range(1, 9):
        x = np.abs(rng.normal(0, 3, 300)).astype(np.float32) + 0.01
        got = ref.minimal_i_given_xb(torch.from_numpy(x), torch.full((len(x),), float(b)), symmetric=True).numpy()
        assert np.all(x <= 2.0**got * (1 - 2.0**-b) * (1 + 1e-5))
        assert np.all(x > 2.0 ** (got - 1) * (1 - 2.0**-b) * (1 - 1e-5))
    # non-symmetric: b <= 0 gives 32
    got = ref.minimal_i_given_xb(torch.tensor([1.0, 2.0]), torch.tensor([0.0, -1.0]), symmetric=False)
    assert got.tolist() == [32.0, 32.0]


@pytest.mark.parametrize('overflow_mode', ('SAT', 'SAT_SYM'))
def test_clip_bound_gradients_match_finite_differences(overflow_mode):
    """The i / f gradients of a saturated output are those of the active bound, a smooth
    function of (i, f); checked by central differences in float64 on that bound."""
    q = fp.get_fixed_quantizer('RND', overflow_mode)
    x = torch.tensor([100.0, -100.0, 0.3, -0.3, 100.0, -100.0])
    k = torch.tensor([1.0, 1.0, 1.0, 1.0, 0.0, 0.0])
    i = torch.tensor([2.0, 2.0, 2.0, 2.0, 1.0, 1.0], requires_grad=True)
    f = torch.tensor([3.0, 3.0, 3.0, 3.0, 2.0, 2.0], requires_grad=True)
    xg = x.clone().requires_grad_(True)
    y = q(xg, k, i, f, True, None)
    y.sum().backward()

    def bound(iv, fv, kv, side):
        hi = 2.0**iv - 2.0**-fv
        if side > 0:
            return hi
        return -kv * hi if overflow_mode == 'SAT_SYM' else -kv * 2.0**iv

    h = 1e-6
    for n in range(6):
        iv, fv, kv = float(i[n]), float(f[n]), float(k[n])
        if n in (2, 3):  # inside the range: straight-through, rounding surrogate only
            assert xg.grad[n] == 1.0 and i.grad[n] == 0.0
            assert np.isclose(float(f.grad[n]), -np.log(2) * float(y[n] - x[n]), rtol=1e-6)
            continue
        side = 1 if x[n] > 0 else -1
        di = (bound(iv + h, fv, kv, side) - bound(iv - h, fv, kv, side)) / (2 * h)
        df = (bound(iv, fv + h, kv, side) - bound(iv, fv - h, kv, side)) / (2 * h)
        assert xg.grad[n] == 0.0  # saturated element receives no gradient (reference tests/base.py:330)
        assert np.isclose(float(i.grad[n]), di, rtol=1e-5, atol=1e-7)
        assert np.isclose(float(f.grad[n]), df, rtol=1e-5, atol=1e-7)


def test_saturating_words_with_negative_total_width_are_defined_by_the_bounds():
    """SAT / SAT_SYM in training where i + f < 0 (the word has no bits left): whether the third-party callable clamps i
    against -f cannot be read from the reference tree, so this build DEFINES the case by the reference's own range
    formulas (fixed_point_quantizer.py:107-116) applied as they stand: hi = 2^i - 2^-f may lie below lo, the upper bound
    wins the forward value, and every violated bound hands the upstream gradient to its own i / f derivative.  Hand-worked
    with k = 1, i = -3, f = 2: 2^i = 0.125, 2^-f = 0.25, hi = -0.125; SAT lo = -0.125; SAT_SYM lo = +0.125 (above hi)."""
    ln2 = math.log(2.0)
    x = torch.tensor([0.3, -1.0, 0.0, -0.125], requires_grad=True)   # rounds (RND, f = 2) to 0.25, -1, 0, 0
    g = torch.tensor([1.0, 2.0, -3.0, 0.5])

    def run(mode, k):
        xs = x.detach().clone().requires_grad_(True)
        i = torch.full((4,), -3.0, requires_grad=True)
        f = torch.full((4,), 2.0, requires_grad=True)
        y = fp.get_fixed_quantizer('RND', mode)(xs, torch.full((4,), float(k)), i, f, True, None)
        y.backward(g)
        return y.detach().tolist(), xs.grad.tolist(), i.grad.tolist(), f.grad.tolist()

    # SAT, k = 1: hi = lo = -0.125.  0.25 and 0 are above hi (upper bound, d/di = ln2 2^i, d/df = ln2 2^-f); -1 is below
    # lo (lower bound -2^i: d/di = -ln2 2^i, d/df = 0); nothing passes, so d/dx = 0 everywhere
    y, dx, di, df = run('SAT', 1)
    assert y == [-0.125] * 4 and dx == [0.0] * 4
    assert di == pytest.approx([ln2 * 0.125 * 1.0, -ln2 * 0.125 * 2.0, ln2 * 0.125 * -3.0, ln2 * 0.125 * 0.5], rel=1e-6)
    assert df == pytest.approx([ln2 * 0.25 * 1.0, 0.0, ln2 * 0.25 * -3.0, ln2 * 0.25 * 0.5], rel=1e-6)
    # SAT, k = 0: lo = 0.  -1 is below lo and not above hi: value 0, no bit-width gradient (lo does not depend on i, f)
    y, dx, di, df = run('SAT', 0)
    assert y == [-0.125, 0.0, -0.125, -0.125] and dx == [0.0] * 4
    assert di == pytest.approx([ln2 * 0.125, 0.0, ln2 * 0.125 * -3.0, ln2 * 0.125 * 0.5], rel=1e-6)
    # SAT_SYM, k = 1: lo = -hi = +0.125 > hi.  0.25 is above hi only; -1 below lo only (value lo = +0.125, d lo = -d hi);
    # 0 violates both: the upper bound wins the value and the two bound gradients cancel exactly
    y, dx, di, df = run('SAT_SYM', 1)
    assert y == [-0.125, 0.125, -0.125, -0.125] and dx == [0.0] * 4
    assert di == pytest.approx([ln2 * 0.125, -ln2 * 0.125 * 2.0, 0.0, 0.0], abs=1e-9)
    assert df == pytest.approx([ln2 * 0.25, -ln2 * 0.25 * 2.0, 0.0, 0.0], abs=1e-9)
    # bit-widths shared by the four elements: autograd of the broadcast adds the per-element terms
    i1, f1 = torch.tensor([-3.0], requires_grad=True), torch.tensor([2.0], requires_grad=True)
    fp.get_fixed_quantizer('RND', 'SAT')(x.detach(), torch.ones(4), i1.expand(4), f1.expand(4), True, None).backward(g)
    assert float(i1.grad) == pytest.approx(ln2 * 0.125 * (1.0 - 2.0 - 3.0 + 0.5), rel=1e-6)
    assert float(f1.grad) == pytest.approx(ln2 * 0.25 * (1.0 - 3.0 + 0.5), rel=1e-6)


def test_ebops_known_answers_at_construction():
    """Closed form dense.py:70-80 with the default bit-widths (8 everywhere):
    in*out*64 + 8*out for the four layers of the 16-64-32-32-5 MLP."""
    mlp = ref.RefMLP()
    want = [66048, 131328, 65792, 10280]
    got = [int(layer._compute_ebops((1, layer.kernel.shape[0]))) for layer in mlp.layers]
    assert got == want and sum(got) == 273448


def test_ebops_bruteforce_python_ints():
    g = torch.Generator().manual_seed(5)
    layer = ref.RefMLP(dims=(6, 4)).layers[0]
    with torch.no_grad():
        layer.iq.quantizer._f.copy_(torch.randint(-3, 7, (1, 6), generator=g).float())
        layer.iq.quantizer._i.copy_(torch.randint(-2, 4, (1, 6), generator=g).float())
        layer.kq.quantizer._b.copy_(torch.randint(0, 9, (6, 4), generator=g).float())
        layer.bq.quantizer._b.copy_(torch.randint(0, 9, (4,), generator=g).float())
    bi = [max(0, int(a + b)) for a, b in zip(layer.iq.quantizer._i.flatten().tolist(), layer.iq.quantizer._f.flatten().tolist())]
    bk = layer.kq.quantizer._b.int().tolist()
    bb = layer.bq.quantizer._b.int().tolist()
    want = sum(bi[r] * bk[r][c] for r in range(6) for c in range(4)) + Fraction(sum(bb), 4) * 4
    assert float(layer._compute_ebops((1, 6))) == float(want)


def test_dummy_quantizers_reduce_qdense_to_dense():
    """Reference tests/test_dense.py:31-46: with dummy quantizers QDense == Dense."""
    g = torch.Generator().manual_seed(6)
    w = torch.randn(12, 8, generator=g)
    b = torch.randn(8, generator=g)
    d = ref.RefQuantizer(ref.RefDummyQuantizer())
    layer = ref.RefQDense(w, b, d, d, d, activation='relu', enable_ebops=False)
    x = torch.randn(50, 12, generator=g)
    assert torch.equal(layer(x, training=False), torch.relu(x @ w + b))


def test_kif_wrap_training_state_machine():
    """fixed_point_quantizer.py:401-413: _i <- max(_i - decay, ceil(log2(max|rx| + 2^-f))), no clip."""
    q = ref.default_quantizer('datalane', (None, 3), q_type='kif', overflow_mode='WRAP')
    x = torch.tensor([[0.1, 3.2, -100.0], [0.2, -7.99, 0.0]])
    y = q(x, training=True)
    assert torch.equal(y, torch.floor(x * 64 + 0.5) / 64)
    # col0: max .203125 -> ceil(log2(.21875)) = -2 -> max(1.99,-2)=1.99 ; col1: 7.984375+2^-6 = 8 -> 3 ; col2: 100 -> 7
    assert torch.allclose(q.quantizer._i, torch.tensor([[1.99, 3.0, 7.0]]))
    assert q.quantizer.bits.tolist() == [[8.0, 9.0, 13.0]]


def test_dummy_quantizers_reduce_qbatchnorm_to_batch_normalisation():
    """The oracle's QBatchNormalization with dummy quantizers is the textbook batch normalisation: training output
    (x - mean) / sqrt(var + eps) * gamma + beta with the biased batch variance, and with momentum 0 the inference
    output repeats it (the check the reference makes at tests/test_batchnorm.py:44-59)."""
    g = torch.Generator().manual_seed(7)
    x = torch.randn(6, 8, 5, generator=g) * 2 + 1
    gamma, beta = torch.rand(5, generator=g) + 0.5, torch.randn(5, generator=g)
    q = lambda: ref.RefQuantizer(ref.RefDummyQuantizer(), None, None, None)  # noqa: E731
    bn = ref.RefQBatchNormalization(2, gamma, beta, torch.randn(5, generator=g), torch.rand(5, generator=g) * 8, q(), q(), q(),
                                    momentum=0.0, epsilon=1e-3, enable_ebops=False)
    mean = x.double().mean(dim=(0, 1))
    var = ((x.double() - mean) ** 2).mean(dim=(0, 1))
    want = ((x.double() - mean) / torch.sqrt(var + 1e-3) * gamma.double() + beta.double()).float()
    y_train = bn(x, training=True)
    assert torch.allclose(y_train, want, atol=2e-6), float((y_train - want).abs().max())
    assert torch.allclose(bn.moving_mean, mean.float(), atol=1e-6) and torch.allclose(bn.moving_variance, var.float(), atol=1e-5)
    y_test = bn(x, training=False)
    assert torch.allclose(y_test, want, atol=2e-6)
    # a dropped term shows: without centring the reference puts 1 in beta's place, without scaling gamma is 1
    bn2 = ref.RefQBatchNormalization(2, None, None, torch.zeros(5), torch.ones(5), q(), q(), q(), momentum=0.0, enable_ebops=False)
    y2 = bn2(x, training=True)
    assert torch.allclose(y2, ((x.double() - mean) / torch.sqrt(var + 1e-3) + 1.0).float(), atol=2e-6)


def test_philox4x32_10_known_answers():
    """The three known-answer vectors of the Random123 library (kat_vectors, philox4x32 with 10 rounds)."""
    import numpy as np

    from oracle.fixed_point import philox4x32_10

    cases = [((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
             ((0xffffffff,) * 4, (0xffffffff,) * 2, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
             ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0), (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1))]
    for ctr, key, want in cases:
        got = philox4x32_10([np.array([c], dtype=np.uint64) for c in ctr], [np.uint64(k) for k in key])
        assert tuple(int(w[0]) for w in got) == want
    # vectorised: the blocks of an array are the blocks of its elements
    ctrs = np.arange(5, dtype=np.uint64)
    many = philox4x32_10([ctrs, ctrs * 0, ctrs * 0 + np.uint64(7), ctrs * 0], [np.uint64(3), np.uint64(0)])
    for j in range(5):
        one = philox4x32_10([np.array([j], dtype=np.uint64), np.zeros(1, np.uint64), np.full(1, 7, np.uint64), np.zeros(1, np.uint64)],
                            [np.uint64(3), np.uint64(0)])
        assert [int(w[j]) for w in many] == [int(w[0]) for w in one]


def test_stochastic_rounding_is_floor_or_ceil_unbiased_and_reproducible():
    """S_RND in training: every value is one of the two neighbours on the 2^-f grid, the mean over many draws is the
    input (the defining property of stochastic rounding), a draw is a function of (seed, offset) only, grid points are
    fixed points, and outside training the mode is plain RND."""
    from oracle.fixed_point import SeedGenerator, get_fixed_quantizer, stochastic_uniform

    u = stochastic_uniform(100001, 12345, 1)
    assert float(u.min()) >= 0.0 and float(u.max()) < 1.0 and abs(float(u.double().mean()) - 0.5) < 5e-3
    assert torch.equal(u[:4097], stochastic_uniform(4097, 12345, 1))  # a prefix does not depend on the length
    assert not torch.equal(u[:64], stochastic_uniform(64, 12345, 2)[:64])

    q = get_fixed_quantizer('S_RND', 'WRAP')
    assert q.stochastic and q.round_mode == 'RND'
    x = torch.tensor([0.3, -1.26, 2.0, 0.125]).repeat(20000, 1)
    f = torch.full_like(x, 2.0)
    gen = SeedGenerator(7)
    y = q.round(x, f, True, gen)
    lo = torch.floor(x * 4) / 4
    assert bool(((y == lo) | (y == lo + 0.25)).all())
    assert bool((y[:, 2] == 2.0).all())  # already on the grid
    assert torch.allclose(y.double().mean(0), x[0].double(), atol=4e-3)
    assert torch.equal(q.round(x, f, True, (7, 1)), y) and gen.offset == 1
    assert not torch.equal(q.round(x, f, True, gen), y)  # the generator has moved on
    k, i = torch.ones_like(x), torch.full_like(x, 3.0)
    assert torch.equal(q(x, k, i, f, False, gen), get_fixed_quantizer('RND', 'WRAP')(x, k, i, f, False, None))
    # surrogate gradient of the draw that was made: d/df = -ln2 * (y - x), d/dx = 1
    xg, fg = x[:8].clone().requires_grad_(True), f[:8].clone().requires_grad_(True)
    yy = q.round(xg, fg, True, (7, 1))
    yy.sum().backward()
    assert torch.equal(xg.grad, torch.ones_like(xg))
    assert torch.allclose(fg.grad, -math.log(2.0) * (yy.detach() - xg.detach()), rtol=1e-6, atol=0)
