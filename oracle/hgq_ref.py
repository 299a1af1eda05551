"""Oracle (test infrastructure, never shipped): the reference's own Python, restated.

Eager fp32 torch-CPU, one torch op per ``keras.ops`` call, autograd backward - i.e. the
way the reference executes on its PyTorch backend (nothing is compiled there, reference
docs/status.md:16).  Doubles as the ``cpu_baseline`` ("port") of ``bench.py``.

Every class cites the reference file:line it follows (paths relative to the reference
root, ``fpq.py`` = src/hgq/quantizer/internal/fixed_point_quantizer.py).

State lives in plain tensors (``_k`` uint8, ``_i``, ``_f`` / ``_b`` fp32) so a test can
copy the product's variables in and compare the variables after a call.

Keras behaviours assumed here that are not in the reference tree: ``keras.backend.epsilon()``
is 1e-7; ``training`` propagates into nested layer calls; ``add_loss`` terms and variable
regularizers are summed into the loss; constraints are applied after the optimizer update.
"""

from __future__ import annotations

from math import prod

import numpy as np
import torch
import torch.nn.functional as F

from .fixed_point import SeedGenerator, get_fixed_quantizer, round_conv

EPSILON = 1e-7  # keras.backend.epsilon() default

# Checker precision.  False: every op in fp32, as the reference executes (this is what ``cpu_baseline`` times).
# True: the contractions (matmul / einsum / convolution) and everything downstream of them are evaluated in float64,
# while every quantizer still sees and produces fp32 values; a parity test that compares sums over 10^5..10^7 terms
# sets it so that its tolerance measures the kernel under test and not the fp32 summation order of this file.
ACC64 = False
# True: every quantizer call keeps its result (with ``retain_grad``) in ``quantizer.taps``, so that a test can bound the
# sum of |terms| behind a bit-width gradient (|term| <= ln2 * 2^-f * |upstream gradient|) and state its tolerance
# relative to that sum instead of to the cancelled total.
TAP_GRADS = False


def _acc(t):
    return t.double() if ACC64 else t


def _f32(t):
    """Operand of a quantizer: always fp32 (a float64 intermediate is rounded once, like the fp32 op would)."""
    return t.float() if t.dtype == torch.float64 else t


# --------------------------------------------------------------------------------------
# fpq.py:16-31
# --------------------------------------------------------------------------------------
def minimal_i_given_xb(x, b, symmetric=False):
    eps = EPSILON
    if symmetric:
        return torch.ceil(torch.log2((x + eps) / (1 - 2.0**-b + eps)))
    i_pos = torch.ceil(torch.log2((x + eps) / (1 - 2.0**-b + eps)))
    i_neg = torch.ceil(torch.log2(-x - eps))
    return torch.where(b > 0, torch.where(x >= 0, i_pos, i_neg), torch.full_like(i_pos, 32.0))


def minimal_i_given_xf(x, f, symmetric=False):
    eps = EPSILON
    if symmetric:
        return torch.ceil(torch.log2(torch.abs(x) + 2**-f))
    i_pos = torch.ceil(torch.log2(x + 2**-f))
    i_neg = torch.ceil(torch.log2(-x - eps))
    return torch.where(x >= 0, i_pos, i_neg)


# --------------------------------------------------------------------------------------
# src/hgq/quantizer/internal/base.py:148-196  DefaultBitwidthMapper
# --------------------------------------------------------------------------------------
class BitwidthMapper:
    def __init__(self, heterogeneous_axis=None, homogeneous_axis=None):
        assert (heterogeneous_axis is None) ^ (homogeneous_axis is None)
        self.heterogeneous_axis = heterogeneous_axis
        self.homogeneous_axis = homogeneous_axis

    def inference_weight_shape(self, input_shape):
        n = len(input_shape)
        axis = list(range(n))
        norm = lambda ax: [a if a >= 0 else a + n for a in ax]  # noqa: E731
        if self.heterogeneous_axis is not None:
            self.heterogeneous_axis = tuple(norm(self.heterogeneous_axis))
            self.homogeneous_axis = tuple(a for a in axis if a not in self.heterogeneous_axis)
        else:
            self.homogeneous_axis = tuple(norm(self.homogeneous_axis))
            self.heterogeneous_axis = tuple(a for a in axis if a not in self.homogeneous_axis)
        shape = [1] * n
        for a in self.heterogeneous_axis:
            assert input_shape[a] is not None
            shape[a] = input_shape[a]
        return tuple(shape)

    def bw_to_x(self, bw, x_shape):
        return torch.broadcast_to(bw, tuple(x_shape))

    def x_to_bw_absmax(self, x):
        if len(self.homogeneous_axis) == 0:
            return torch.abs(x)
        return torch.amax(torch.abs(x), dim=self.homogeneous_axis, keepdim=True)

    def x_to_bw_sign(self, x):
        neg = x < 0
        for a in self.homogeneous_axis:
            neg = torch.any(neg, dim=a, keepdim=True)
        return neg


def _clip_constraint(c, w):
    """constraints/__init__.py:19-21 (MinMax), :37-39 (Constant), :51-53 (Min), :65-67 (Max)."""
    if c is None:
        return w
    kind = c[0]
    if kind == 'minmax':
        return torch.clamp(w, c[1], c[2])
    if kind == 'min':
        return torch.clamp(w, min=c[1])
    if kind == 'max':
        return torch.clamp(w, max=c[1])
    if kind == 'constant':
        return torch.full_like(w, c[1])
    raise ValueError(kind)


class RefFixedPointQuantizer:
    """fpq.py:34-150 (base), :153-307 (KBI), :310-459 (KIF).

    ``q_type`` is 'kif' or 'kbi'.  Constraints are ('minmax', lo, hi) tuples or None;
    regularizers are the MonoL1 coefficient or None.
    """

    def __init__(
        self,
        q_type,
        input_shape,
        *,
        k0=1,
        i0=2,
        f0=6,
        b0=8,
        round_mode='RND',
        overflow_mode='WRAP',
        ic=None,
        fc=None,
        bc=None,
        ir=None,
        fr=None,
        br=None,
        i_decay_speed=float('inf'),
        homogeneous_axis=None,
        heterogeneous_axis=None,
        is_weight=False,
        trainable=True,
        seed=0,
    ):
        self.q_type = q_type
        self.round_mode = round_mode.upper()
        self.overflow_mode = overflow_mode.upper()
        self.symmetric = self.overflow_mode.endswith('SYM')
        self.is_weight = is_weight
        self.trainable = trainable
        self.bw_mapper = BitwidthMapper(heterogeneous_axis, homogeneous_axis)
        self.q = get_fixed_quantizer(self.round_mode, self.overflow_mode)
        self.seed_gen = SeedGenerator(seed) if self.q.stochastic else None  # fpq.py:56-57
        shape = self.bw_mapper.inference_weight_shape(tuple(input_shape))
        self._k = torch.full(shape, int(k0), dtype=torch.uint8)
        i_trainable = self.overflow_mode != 'WRAP'
        self._i = torch.full(shape, float(i0)).requires_grad_(i_trainable and trainable)
        if q_type == 'kif':
            self._f = torch.full(shape, float(f0)).requires_grad_(trainable)
            self._b = None
        else:
            self._b = torch.full(shape, float(b0)).requires_grad_(trainable)
            self._f = None
        self.i_constraint, self.f_constraint, self.b_constraint = ic, fc, bc
        self.i_regularizer, self.f_regularizer, self.b_regularizer = ir, fr, br
        self.i_decay_speed = torch.tensor(float(i_decay_speed))

    # ---- properties: fpq.py:244-265 (KBI), :431-449 (KIF)
    @property
    def k(self):
        return self._k.to(torch.float32)

    @property
    def i(self):
        return round_conv(self._i)

    @property
    def f(self):
        if self.q_type == 'kif':
            return round_conv(self._f)
        return self.b - self.i

    @property
    def b(self):
        if self.q_type == 'kif':
            return torch.relu(self.i + self.f)
        return round_conv(self._b)

    @property
    def kif(self):
        if self.q_type == 'kif':
            return self.k, self.i, self.f
        k, b, i = self.k, self.b, self.i
        return k, i, b - i

    # ---- fpq.py:92-120
    @property
    def bits(self):
        return self.b if self.overflow_mode != 'SAT' else self.b + self.k

    @property
    def fbits(self):
        b = self.b
        if self.overflow_mode == 'WRAP':
            return b + self.k * (b > 0).to(torch.float32)
        return b + self.k

    @property
    def min(self):
        if self.symmetric:
            return -self.k * (2.0**self.i - 2.0**-self.f)
        return -self.k * (2.0**self.i)

    @property
    def max(self):
        return 2.0**self.i - 2.0**-self.f

    @property
    def epsilon(self):
        return 2.0**-self.f

    def variables(self):
        out = {'_k': self._k, '_i': self._i}
        if self.q_type == 'kif':
            out['_f'] = self._f
        else:
            out['_b'] = self._b
        return out

    def trainable_variables(self):
        return [v for v in (self._i, self._f, self._b) if v is not None and v.requires_grad]

    def regularization_loss(self):
        """regularizers/__init__.py:13-14 applied to each trainable variable that carries one
        (Keras collects regularization losses from trainable weights only)."""
        loss = 0.0
        for v, r in ((self._i, self.i_regularizer), (self._f, self.f_regularizer), (self._b, self.b_regularizer)):
            if v is not None and r is not None and v.requires_grad:
                loss = loss + r * torch.sum(v)
        return loss

    def apply_constraints(self):
        with torch.no_grad():
            for v, c in ((self._i, self.i_constraint), (self._f, self.f_constraint), (self._b, self.b_constraint)):
                if v is not None and c is not None and v.requires_grad:
                    v.copy_(_clip_constraint(c, v))

    # ---- fpq.py:142-150
    def _base_call(self, x, training):
        k, i, f = self.kif
        k = self.bw_mapper.bw_to_x(k, x.shape)
        i = self.bw_mapper.bw_to_x(i, x.shape)
        f = self.bw_mapper.bw_to_x(f, x.shape)
        ret = self.q(x, k, i, f, training is True, self.seed_gen)
        if not training:
            ret = torch.where(k + i + f > 0, ret, torch.zeros_like(ret))
        return ret

    def call(self, x, training=None):
        if self.q_type == 'kif':
            return self._call_kif(x, training)
        return self._call_kbi(x, training)

    # ---- fpq.py:401-429
    def _call_kif(self, x, training):
        if self.overflow_mode == 'WRAP' and self.trainable:
            f = self.bw_mapper.bw_to_x(self.f, x.shape)
            stochastic = self.q.stochastic and training is True  # fpq.py:404
            rx = self.q.round(x, f, stochastic, self.seed_gen)
            if training or training == 'tracing':
                xr = self.bw_mapper.x_to_bw_absmax(rx.detach())
                _new_i = minimal_i_given_xf(xr, self.f.detach(), self.symmetric)
                with torch.no_grad():
                    if training:
                        # the constraint is applied to a dead value in the reference (:411-412)
                        new_i = torch.maximum(self._i - self.i_decay_speed, _new_i)
                        self._i.copy_(new_i)
                    else:
                        _new_i = _clip_constraint(self.i_constraint, _new_i)
                        new_i = torch.maximum(self.i.detach(), _new_i)
                        new_k = self.bw_mapper.x_to_bw_sign(rx.detach())
                        self._k.copy_((self._k.bool() | new_k).to(torch.uint8))
                        self._i.copy_(new_i)
                return rx
            if self.is_weight:
                return rx
        return self._base_call(x, training is True)

    # ---- fpq.py:277-307
    def _call_kbi(self, x, training):
        if self.overflow_mode == 'WRAP' and self.trainable:
            if training or training == 'tracing':
                xr = self.bw_mapper.x_to_bw_absmax(x.detach())
                new_i = minimal_i_given_xb(xr, self.b.detach(), self.symmetric)
                if training:
                    with torch.no_grad():
                        new_i = torch.maximum(self._i - self.i_decay_speed, new_i)
                        new_i = _clip_constraint(self.i_constraint, new_i)
                        self._i.copy_(new_i)
                    f = self.bw_mapper.bw_to_x(self.f, x.shape)
                    return self.q.round(x, f, self.q.stochastic, self.seed_gen)  # fpq.py:279,288
                with torch.no_grad():
                    new_i = torch.maximum(self.i.detach(), new_i)
                    new_i = _clip_constraint(self.i_constraint, new_i)
                f = self.bw_mapper.bw_to_x(self.b - new_i, x.shape)
                rx = self.q.round(x, f, False, None)
                with torch.no_grad():
                    new_k = self.bw_mapper.x_to_bw_sign(rx.detach()) & (self.b.detach() > 0)
                    self._k.copy_((self._k.bool() | new_k).to(torch.uint8))
                    self._i.copy_(new_i)
                return rx
            if self.is_weight:
                f = self.bw_mapper.bw_to_x(self.f, x.shape)
                if self.q.round_mode == 'RND':
                    return self.q.round(x, f, False, None)
        return self._base_call(x, training is True)


class RefDummyQuantizer:
    """src/hgq/quantizer/internal/base.py:118-145."""

    q_type = 'dummy'

    def __init__(self):
        self.bw_mapper = BitwidthMapper(None, ())

    def call(self, x, training=None):
        return x

    @property
    def bits(self):
        return torch.tensor(0.0)

    fbits = bits

    def trainable_variables(self):
        return []

    def regularization_loss(self):
        return 0.0

    def apply_constraints(self):
        pass


class RefQuantizer:
    """src/hgq/quantizer/quantizer.py:11-104: scaler / qnoise / affine wrapper."""

    def __init__(self, inner, scaler=None, affine=None, qnoise_factor=None):
        self.quantizer = inner
        self.scaler, self.affine, self.qnoise_factor = scaler, affine, qnoise_factor

    def __call__(self, x, training=None):
        inputs = x
        if self.scaler is not None:
            inputs = inputs / self.scaler
        out = self.quantizer.call(inputs, training=training)
        if TAP_GRADS and out.requires_grad:  # a test wants the upstream gradient of every quantizer call afterwards
            out.retain_grad()
            self.quantizer.taps = getattr(self.quantizer, 'taps', []) + [out]
        if self.scaler is not None:
            out = out * self.scaler
        if self.qnoise_factor is not None and training:
            out = inputs + self.qnoise_factor * (out - inputs)
        if self.affine is not None:
            out = out * self.affine[0] + self.affine[1]
        return out

    @property
    def bits(self):
        return self.quantizer.bits

    def bits_(self, shape):
        return self.quantizer.bw_mapper.bw_to_x(self.bits, tuple(shape))


# --------------------------------------------------------------------------------------
# layers
# --------------------------------------------------------------------------------------
class RefQLayer:
    """src/hgq/layers/core/base.py:57-116 (the ``call`` wrapper) and :119-243."""

    enable_ebops = True
    ebops_factor = 1.0
    oq = None

    def _init_common(self, beta0=1e-5, enable_ebops=True):
        self.enable_ebops = enable_ebops
        self.beta = torch.tensor(float(beta0))
        self.ebops_value = torch.zeros((), dtype=torch.int64)  # the uint32 `_ebops` variable
        self.losses = []

    def quantizers(self):
        raise NotImplementedError

    def __call__(self, x, training=None):
        self.losses = []
        r = self.call(x, training=training)
        if (training or training == 'tracing') and self.enable_ebops:
            shape = (1,) + tuple(x.shape[1:])
            ebops = self._compute_ebops(shape) * self.ebops_factor
            # ops.cast(float -> uint32) truncates toward zero (core/base.py:103)
            self.ebops_value = ebops.detach().to(torch.int64)
            self.losses.append(ebops * self.beta)
        if self.oq is not None:
            r = self.oq(r, training=training)
        return r

    def extra_loss(self):
        loss = 0.0
        for term in self.losses:
            loss = loss + term
        for q in self.quantizers():
            loss = loss + q.quantizer.regularization_loss()
        return loss

    def trainable_variables(self):
        out = list(self.weights())
        for q in self.quantizers():
            out += q.quantizer.trainable_variables()
        return out

    def apply_constraints(self):
        for q in self.quantizers():
            q.quantizer.apply_constraints()


class RefQDense(RefQLayer):
    """src/hgq/layers/core/dense.py:12-102."""

    def __init__(self, kernel, bias, iq, kq, bq, activation=None, beta0=1e-5, enable_ebops=True,
                 parallelization_factor=-1, n_parallel=1, oq=None):
        self._init_common(beta0, enable_ebops and iq is not None)
        self.kernel = kernel.detach().clone().requires_grad_(True)
        self.bias = None if bias is None else bias.detach().clone().requires_grad_(True)
        self.iq, self.kq, self.bq, self.oq = iq, kq, bq, oq
        self.activation = activation
        self.n_parallel = n_parallel
        self.parallelization_factor = parallelization_factor if parallelization_factor >= 0 else n_parallel

    def weights(self):
        return [w for w in (self.kernel, self.bias) if w is not None]

    def quantizers(self):
        return [q for q in (self.iq, self.kq, self.bq, self.oq) if q is not None]

    def call(self, x, training=None):
        if self.iq is not None:
            x = self.iq(x, training=training)
        qkernel = self.kq(self.kernel, training=training)
        y = torch.matmul(_acc(x), _acc(qkernel))
        if self.bias is not None:
            y = y + self.bq(self.bias, training=training)
        if self.activation == 'relu':
            y = torch.relu(y)
        elif self.activation is not None:
            raise ValueError(self.activation)
        return y

    def _compute_ebops(self, shape):
        bw_inp = self.iq.bits_(shape)
        bw_ker = self.kq.bits_(self.kernel.shape)
        ebops = torch.sum(torch.matmul(bw_inp, bw_ker))
        if self.bq is not None:
            bw_bias = self.bq.bits_(self.bias.shape)
            size = float(prod(shape[:-1]) * self.kernel.shape[-1])
            ebops = ebops + torch.mean(bw_bias) * size
        return ebops * self.parallelization_factor / self.n_parallel


def _einsum_free0_size(equation, input_shape):
    """src/hgq/layers/core/einsum_dense.py:10-20."""
    _inp, _ker_out = equation.split(',', 1)
    _ker, _out = _ker_out.split('->', 1)
    n_parallel = 1
    for ax, dim in zip(_inp[1:], input_shape[1:]):
        if ax not in _ker and ax in _out:
            n_parallel *= dim
    return n_parallel


class RefQEinsumDense(RefQLayer):
    """src/hgq/layers/core/einsum_dense.py:23-115."""

    def __init__(self, equation, kernel, bias, iq, kq, bq, input_shape, out_shape_tail, activation=None,
                 beta0=1e-5, enable_ebops=True, parallelization_factor=-1, oq=None):
        self._init_common(beta0, enable_ebops and iq is not None)
        self.equation = equation
        self.kernel = kernel.detach().clone().requires_grad_(True)
        self.bias = None if bias is None else bias.detach().clone().requires_grad_(True)
        self.iq, self.kq, self.bq, self.oq = iq, kq, bq, oq
        self.activation = activation
        self.n_parallel = _einsum_free0_size(equation, input_shape)
        self.parallelization_factor = parallelization_factor if parallelization_factor >= 0 else self.n_parallel
        self.ebops_equation = equation.split('->')[0] + '->'
        self.out_size = prod(out_shape_tail)  # prod(full_output_shape[1:])

    def weights(self):
        return [w for w in (self.kernel, self.bias) if w is not None]

    def quantizers(self):
        return [q for q in (self.iq, self.kq, self.bq, self.oq) if q is not None]

    def call(self, x, training=None):
        qkernel = self.kq(self.kernel, training=training)
        if self.iq is not None:
            x = self.iq(x, training=training)
        y = torch.einsum(self.equation, _acc(x), _acc(qkernel))
        if self.bias is not None:
            y = y + self.bq(self.bias, training=training)
        if self.activation == 'relu':
            y = torch.relu(y)
        elif self.activation is not None:
            raise ValueError(self.activation)
        return y

    def _compute_ebops(self, shape):
        bw_inp = self.iq.bits_(shape)
        bw_ker = self.kq.bits_(self.kernel.shape)
        ebops = torch.einsum(self.ebops_equation, bw_inp, bw_ker)
        if self.bq is not None:
            bw_bias = self.bq.bits_(self.bias.shape)
            ebops = ebops + torch.mean(bw_bias) * float(self.out_size)
        return ebops * self.parallelization_factor / self.n_parallel


class RefQEinsumDenseBatchnorm(RefQEinsumDense):
    """src/hgq/layers/einsum_dense_batchnorm.py:11-211.  ``moments`` is restated as Keras' torch
    backend computes it: mean, and mean(x**2) - mean**2 (biased variance)."""

    def __init__(self, *args, gamma, moving_mean, moving_variance, normalize_axes, momentum=0.99, **kwargs):
        super().__init__(*args, **kwargs)
        self.gamma = None if gamma is None else gamma.detach().clone().requires_grad_(True)
        self.moving_mean = moving_mean.detach().clone()
        self.moving_variance = moving_variance.detach().clone()
        self.momentum = momentum
        kernel_axes, output_axes = self.equation.split(',')[1].split('->')
        norm = ''.join(c for c in kernel_axes if c in normalize_axes)
        self.reduction_axes = tuple(i for i, c in enumerate(output_axes) if c not in norm)
        self.fused_kernel_equation = f'{kernel_axes},{norm}->{kernel_axes}'
        first = min(output_axes.find(c) for c in normalize_axes)
        self.norm_axes_spec = output_axes[first:]
        self.normalize_axes = normalize_axes

    def weights(self):
        return super().weights() + ([self.gamma] if self.gamma is not None else [])

    def fused(self, training, mean, var):
        gamma = self.gamma if self.gamma is not None else 1
        scaler = gamma / torch.sqrt(var + EPSILON)
        fused_kernel = torch.einsum(self.fused_kernel_equation, _acc(self.kernel), scaler)
        qkernel = self.kq(_f32(fused_kernel), training=training)
        offset = torch.reshape(-mean * scaler, self.bias.shape)
        qbias = self.bq(_f32(self.bias + offset), training=training)
        return qkernel, qbias

    def call(self, x, training=None):
        if self.iq is not None:
            x = self.iq(x, training=training)
        if training:
            z = torch.einsum(self.equation, _acc(x), _acc(self.kernel))
            mean = torch.mean(z, dim=self.reduction_axes)
            var = torch.mean(torch.square(z), dim=self.reduction_axes) - torch.square(mean)
            with torch.no_grad():
                self.moving_mean.copy_(self.moving_mean * self.momentum + mean * (1.0 - self.momentum))
                self.moving_variance.copy_(self.moving_variance * self.momentum + var * (1.0 - self.momentum))
        else:
            var, mean = self.moving_variance, self.moving_mean
        qkernel, qbias = self.fused(training, mean, var)
        y = torch.einsum(self.equation, _acc(x), _acc(qkernel)) + qbias
        if self.activation == 'relu':
            y = torch.relu(y)
        return y


class RefQBatchNormalization(RefQLayer):
    """src/hgq/layers/batch_normalization.py:10-206 on top of Keras' BatchNormalization: moments are mean and
    mean(x**2) - mean**2 over all axes but ``axis`` (the torch backend's ``moments``); the layer's own epsilon;
    ``center=False`` puts 1 in the place of ``bn_beta`` (:117-120, :145-148)."""

    def __init__(self, axis, gamma, beta_bn, moving_mean, moving_variance, iq, kq, bq, momentum=0.99, epsilon=1e-3, beta0=1e-5,
                 enable_ebops=True):
        self._init_common(beta0, enable_ebops)
        self.axis, self.momentum, self.epsilon = axis, momentum, epsilon
        self.gamma = None if gamma is None else gamma.detach().clone().requires_grad_(True)
        self.bn_beta = None if beta_bn is None else beta_bn.detach().clone().requires_grad_(True)
        self.moving_mean, self.moving_variance = moving_mean.detach().clone(), moving_variance.detach().clone()
        self.iq, self.kq, self.bq = iq, kq, bq

    def weights(self):
        return [w for w in (self.gamma, self.bn_beta) if w is not None]

    def quantizers(self):
        return [q for q in (self.iq, self.kq, self.bq) if q is not None]

    def _bshape(self, x):
        shape = [1] * x.dim()
        shape[self.axis] = x.shape[self.axis]
        return shape

    def call(self, x, training=None):
        if self.iq is not None:
            x = self.iq(x, training=training)
        if training:
            axes = tuple(a for a in range(x.dim()) if a != self.axis % x.dim())
            mean = torch.mean(x, dim=axes)
            var = torch.mean(torch.square(x), dim=axes) - torch.square(mean)
            with torch.no_grad():
                self.moving_mean.copy_(self.moving_mean * self.momentum + mean * (1.0 - self.momentum))
                self.moving_variance.copy_(self.moving_variance * self.momentum + var * (1.0 - self.momentum))
        else:
            mean, var = self.moving_mean, self.moving_variance
        gamma = self.gamma if self.gamma is not None else 1
        bn_beta = self.bn_beta if self.bn_beta is not None else 1
        scale = gamma / torch.sqrt(var + self.epsilon)
        offset = bn_beta - mean * scale
        qscale = torch.reshape(self.kq(scale, training=training), self._bshape(x))
        qoffset = torch.reshape(self.bq(offset, training=training), self._bshape(x))
        return x * qscale + qoffset

    def _compute_ebops(self, shape):
        bshape = [1] * len(shape)
        bshape[self.axis] = shape[self.axis]
        bw_inp = self.iq.bits_(shape)
        bw_ker = torch.reshape(self.kq.bits_(self.moving_mean.shape), bshape)
        bw_bias = torch.reshape(self.bq.bits_(self.moving_mean.shape), bshape)
        size = float(np.prod(shape))
        return torch.sum(bw_inp * bw_ker) + torch.mean(bw_bias) * size


class RefQUnaryFunctionLUT(RefQLayer):
    """src/hgq/layers/activation.py:18-67."""

    def __init__(self, fn, iq, oq, beta0=1e-5, enable_ebops=True):
        self._init_common(beta0, enable_ebops)
        self.fn, self.iq, self.oq = fn, iq, oq

    def weights(self):
        return []

    def quantizers(self):
        return [q for q in (self.iq, self.oq) if q is not None]

    def call(self, x, training=None):
        if self.iq is not None:
            x = self.iq(x, training=training)
        return self.fn(x)

    def _compute_ebops(self, shape):
        bw_inp = self.iq.bits_(shape)
        bw_out = self.oq.bits_(shape)
        return torch.sum((2.0**bw_inp) * bw_out) * 1e-4


class RefQSoftmax(RefQLayer):
    """src/hgq/layers/softmax.py:13-161.  ``stable`` False is the form without the max subtraction (:116-120): the
    exp table then has no input quantizer and no EBOPs of its own (:87-96) and its function is exp(+x * scaler) (:49-53)."""

    def __init__(self, axes, exp_table, inv_table, oq, iq=None, input_scaler=1.0, beta0=1e-5, enable_ebops=True,
                 parallelization_factor=-1, stable=True):
        self._init_common(beta0, enable_ebops)
        self.stable = stable
        self.axes = tuple(axes)
        self.exp_table, self.inv_table, self.oq, self.iq = exp_table, inv_table, oq, iq
        self.input_scaler = input_scaler
        self.parallelization_factor = parallelization_factor

    def weights(self):
        return []

    def quantizers(self):
        return [q for q in (self.iq, self.oq) if q is not None] + self.exp_table.quantizers() + self.inv_table.quantizers()

    def __call__(self, x, training=None, mask=None):
        self._mask = mask
        return super().__call__(x, training=training)

    def call(self, x, training=None):
        mask = self._mask
        if self.iq is not None:
            x = self.iq(x, training=training)
        if self.stable:
            if mask is not None:
                x = mask.to(x.dtype) * x - (1 - mask.to(x.dtype)) * 1e9
            x = torch.amax(x, dim=self.axes, keepdim=True) - x
        e = self.exp_table(x, training=training)
        if mask is not None:
            e = mask.to(x.dtype) * e
        s = torch.sum(e, dim=self.axes, keepdim=True)
        return e * self.inv_table(s, training=training)

    def extra_loss(self):
        return super().extra_loss() + sum(t for t in self.exp_table.losses) + sum(t for t in self.inv_table.losses)

    def _compute_ebops(self, shape):
        accum_shape = tuple(1 if i in self.axes else s for i, s in enumerate(shape))
        max_instance = prod(accum_shape)
        n_instance = self.parallelization_factor if self.parallelization_factor > 0 else max_instance
        factor = n_instance / max_instance
        inp_bits = self.iq.bits_(shape) if self.iq is not None else 0
        exp_bits = self.exp_table.oq.bits_(shape)
        inv_bits = self.inv_table.oq.bits_(accum_shape)
        if self.stable:
            sub = torch.sum(inp_bits) if self.iq is not None else torch.sum(self.exp_table.iq.bits_(shape))
        else:
            sub = 0.0
        accum = torch.sum(exp_bits) - torch.sum(torch.amin(exp_bits, dim=self.axes))
        mult = torch.sum(exp_bits * inv_bits)
        ebops = sub + accum + mult
        if not self.stable:  # the exp table has no input quantizer of its own: its size is counted here (:150-152)
            ebops = ebops + torch.sum((2.0**inp_bits) * exp_bits) * 1e-4
        return ebops * factor


def keras_attention_equations(rank, attn_axes):
    """The einsum strings Keras' multi-head attention builds for projected tensors of ``rank`` axes
    [batch, seq..., heads, channels] (the reference imports the builder at src/hgq/layers/attn/mha.py:10 and uses its
    result at :315-319): query axes are lettered a, b, c, ...; the key / value side reuses the query's letter on every
    axis that is not attended and on the last axis, and takes the next unused letters on the attended ones; scores are
    [kept axes..., attended query axes..., attended key axes...]."""
    letters = 'abcdefghijklmnopqrstuvwxyz'
    target = letters[:rank]
    kept = tuple(i for i in range(rank) if i not in tuple(attn_axes) + (rank - 1,))
    nxt, source = rank, ''
    for i in range(rank):
        if i in kept or i == rank - 1:
            source += target[i]
        else:
            source += letters[nxt]
            nxt += 1
    product = ''.join([target[i] for i in kept] + [target[i] for i in attn_axes] + [source[i] for i in attn_axes])
    return '%s,%s->%s' % (source, target, product), '%s,%s->%s' % (product, source, target)


class RefQMultiHeadAttention(RefQLayer):
    """src/hgq/layers/attn/mha.py:27-537 for inputs [batch, seq..., features] attending over all sequence axes."""

    def __init__(self, query_dense, key_dense, value_dense, output_dense, softmax, beta0=1e-5, enable_ebops=True,
                 parallelization_factor=-1):
        self._init_common(beta0, enable_ebops)
        self.qd, self.kd, self.vd, self.od, self.softmax = query_dense, key_dense, value_dense, output_dense, softmax
        self.parallelization_factor = parallelization_factor

    def sublayers(self):
        return [self.qd, self.kd, self.vd, self.softmax, self.softmax.exp_table, self.softmax.inv_table, self.od]

    def weights(self):
        return [w for l in (self.qd, self.kd, self.vd, self.od) for w in l.weights()]

    def quantizers(self):
        seen, out = set(), []
        for l in (self.qd, self.kd, self.vd, self.od, self.softmax):
            for q in l.quantizers():
                if id(q) not in seen:
                    seen.add(id(q))
                    out.append(q)
        return out

    def call(self, x, value=None, key=None, training=None, mask=None):
        value = x if value is None else value  # mha.py:452-455
        key = value if key is None else key
        q = self.qd(x, training=training)
        k = self.kd(key, training=training)
        v = self.vd(value, training=training)
        rank = q.dim()
        attn_axes = tuple(range(1, rank - 2))  # mha.py:312-313
        self._dot_eq, self._combine_eq = keras_attention_equations(rank, attn_axes)
        scores = torch.einsum(self._dot_eq, k, q * 1.0)  # mha.py:521-525 (the 1/sqrt(d) factor sits in the softmax)
        m = mask
        if m is not None:  # Keras' _masked_softmax: new axes ahead of the attended ones until the ranks agree
            while m.dim() < scores.dim():
                m = m.unsqueeze(-2 * len(attn_axes) - 1)
        scores = self.softmax(scores, training=training, mask=m)
        out = torch.einsum(self._combine_eq, scores, v)  # mha.py:536
        self._shapes = (q.shape, k.shape, v.shape, scores.shape)
        return self.od(out, training=training)

    def __call__(self, x, value=None, key=None, training=None, mask=None):
        self.losses = []
        r = self.call(x, value, key, training=training, mask=mask)
        if (training or training == 'tracing') and self.enable_ebops:
            ebops = self._compute_ebops()
            self.ebops_value = ebops.detach().to(torch.int64)
            self.losses.append(ebops * self.beta)
        return r

    def extra_loss(self):
        loss = 0.0
        for term in self.losses:
            loss = loss + term
        for l in (self.qd, self.kd, self.vd, self.od, self.softmax, self.softmax.exp_table, self.softmax.inv_table):
            for term in l.losses:
                loss = loss + term
        for q in self.quantizers():
            loss = loss + q.quantizer.regularization_loss()
        return loss

    def _compute_ebops(self):
        qs, ks, vs, ss = ((1,) + tuple(s[1:]) for s in self._shapes)
        bw_q, bw_k, bw_v = self.qd.oq.bits_(qs), self.kd.oq.bits_(ks), self.vd.oq.bits_(vs)
        bw_attn = self.softmax.oq.bits_(ss)
        # mha.py:386-416 with the strings of :246-247
        dot_eq, combine_eq = keras_attention_equations(len(qs), tuple(range(1, len(qs) - 2)))
        ebops = torch.einsum(dot_eq.split('->')[0] + '->', bw_k, bw_q) + torch.einsum(combine_eq.split('->')[0] + '->', bw_attn, bw_v)
        if self.parallelization_factor > 0:
            return ebops * self.parallelization_factor
        return ebops


class RefQConv2D(RefQLayer):
    """src/hgq/layers/conv.py:12-102: channels-last input, HWIO kernel, 'valid' or 'same' padding."""

    def __init__(self, kernel, bias, iq, kq, bq, strides=(1, 1), padding='valid', activation=None, beta0=1e-5,
                 enable_ebops=True, parallelization_factor=-1, n_parallel=1, oq=None):
        self._init_common(beta0, enable_ebops and iq is not None)
        self.kernel = kernel.detach().clone().requires_grad_(True)
        self.bias = None if bias is None else bias.detach().clone().requires_grad_(True)
        self.iq, self.kq, self.bq, self.oq = iq, kq, bq, oq
        self.strides, self.padding, self.activation = tuple(strides), padding, activation
        self.n_parallel = n_parallel
        self.parallelization_factor = parallelization_factor if parallelization_factor > 0 else n_parallel

    def weights(self):
        return [w for w in (self.kernel, self.bias) if w is not None]

    def quantizers(self):
        return [q for q in (self.iq, self.kq, self.bq, self.oq) if q is not None]

    def conv(self, x, w):
        x = x.permute(0, 3, 1, 2)
        w = w.permute(3, 2, 0, 1).contiguous()  # (a permuted one-filter kernel trips torch's CPU convolution backward)
        if self.padding == 'same':
            pads = []
            for d in (1, 0):
                n, k, st = x.shape[2 + d], w.shape[2 + d], self.strides[d]
                total = max((-(-n // st) - 1) * st + k - n, 0)
                pads += [total // 2, total - total // 2]
            x = F.pad(x, pads)
        return F.conv2d(x, w, None, self.strides).permute(0, 2, 3, 1)

    def call(self, x, training=None):
        if self.iq is not None:
            x = self.iq(x, training=training)
        y = self.conv(_acc(x), _acc(self.kq(self.kernel, training=training)))
        if self.bias is not None:
            y = y + self.bq(self.bias, training=training).reshape(1, 1, 1, -1)
        if self.activation == 'relu':
            y = torch.relu(y)
        return y

    def _compute_ebops(self, shape):
        bw_inp = self.iq.bits_(shape)
        bw_ker = self.kq.bits_(self.kernel.shape)
        ebops = torch.sum(self.conv(bw_inp, bw_ker)) * (self.parallelization_factor / self.n_parallel)
        if self.bq is not None:
            size = float(prod(shape[:-1]) * self.kernel.shape[-1])
            ebops = ebops + torch.mean(self.bq.bits_(self.bias.shape)) * size
        return ebops


class RefQPooling2D(RefQLayer):
    """src/hgq/layers/pooling.py:23-47 on top of MaxPooling2D / AveragePooling2D (channels-last;
    'same' pads like Keras: odd pad after, padding never wins a maximum and is not counted in a mean)."""

    def __init__(self, mode, pool_size, strides, padding, iq, oq=None, beta0=1e-5, enable_ebops=True, parallelization_factor=-1,
                 n_parallel=1):
        self._init_common(beta0, enable_ebops and iq is not None)
        self.mode, self.pool_size, self.strides, self.padding = mode, tuple(pool_size), tuple(strides), padding
        self.iq, self.oq = iq, oq
        self.n_parallel = n_parallel
        self.parallelization_factor = parallelization_factor if parallelization_factor > 0 else n_parallel

    def weights(self):
        return []

    def quantizers(self):
        return [q for q in (self.iq, self.oq) if q is not None]

    def call(self, x, training=None):
        if self.iq is not None:
            x = self.iq(x, training=training)
        x = x.permute(0, 3, 1, 2)
        pads = [0, 0, 0, 0]
        if self.padding == 'same':
            pads = []
            for d in (1, 0):
                n, k, st = x.shape[2 + d], self.pool_size[d], self.strides[d]
                total = max((-(-n // st) - 1) * st + k - n, 0)
                pads += [total // 2, total - total // 2]
        if self.mode == 'max':
            y = F.max_pool2d(F.pad(x, pads, value=float('-inf')), self.pool_size, self.strides)
        else:
            num = F.avg_pool2d(F.pad(x, pads), self.pool_size, self.strides, divisor_override=1)
            cnt = F.avg_pool2d(F.pad(torch.ones_like(x[:1, :1]), pads), self.pool_size, self.strides, divisor_override=1)
            y = num / cnt
        return y.permute(0, 2, 3, 1)

    def _compute_ebops(self, shape):
        return torch.sum(self.iq.bits_(shape)) * self.parallelization_factor / self.n_parallel


# --------------------------------------------------------------------------------------
# the QDense-MLP training step (reference call stack: tests/base.py:302-321 and README.md:57-67)
# --------------------------------------------------------------------------------------
def default_quantizer(place, input_shape, *, q_type, overflow_mode, round_mode='RND', **over):
    """Default configs of src/hgq/quantizer/config.py:75-147,199-205 after a scope set
    ``overflow_mode`` / ``q_type`` for this place."""
    if q_type == 'kbi':
        cfg = dict(k0=1, b0=8, i0=2, round_mode=round_mode, overflow_mode=overflow_mode, br=1e-8, ir=None)
        if place == 'weight':
            cfg.update(bc=('minmax', 0.0, 23.0), i_decay_speed=float('inf'), homogeneous_axis=(), is_weight=True)
        elif place == 'table':
            cfg.update(bc=('minmax', 0.0, 23.0), i_decay_speed=float('inf'), heterogeneous_axis=(), is_weight=False)
        elif place == 'bias':
            cfg.update(bc=('minmax', 0.0, 24.0), i_decay_speed=0.01, homogeneous_axis=(), is_weight=False)
        else:
            cfg.update(bc=('minmax', 0.0, 24.0), i_decay_speed=0.01, homogeneous_axis=(0,), is_weight=False)
    else:
        cfg = dict(k0=1, i0=2, f0=6, round_mode=round_mode, overflow_mode=overflow_mode,
                   ic=('minmax', -23.0, 23.0), fc=('minmax', -24.0, 24.0), ir=1e-8, fr=1e-8)
        if place == 'weight':
            cfg.update(i_decay_speed=float('inf'), homogeneous_axis=(), is_weight=True)
        elif place == 'table':
            cfg.update(i_decay_speed=float('inf'), heterogeneous_axis=(), is_weight=False)
        elif place == 'bias':
            cfg.update(i_decay_speed=0.01, homogeneous_axis=(), is_weight=False)
        else:
            cfg.update(i_decay_speed=0.01, homogeneous_axis=(0,), is_weight=False)
    if over.get('heterogeneous_axis') is not None:
        cfg.pop('homogeneous_axis', None)
    if over.get('homogeneous_axis') is not None:
        cfg.pop('heterogeneous_axis', None)
    cfg.update(over)
    return RefQuantizer(RefFixedPointQuantizer(q_type, input_shape, **cfg))


def glorot_uniform(shape, generator, fan_in=None, fan_out=None):
    fan_in = shape[0] if fan_in is None else fan_in
    fan_out = shape[-1] if fan_out is None else fan_out
    limit = float(np.sqrt(6.0 / (fan_in + fan_out)))
    return (torch.rand(shape, generator=generator) * 2 - 1) * limit


class RefMLP:
    """QDense 16->64->32->32->5 under the README scopes: kbi SAT_SYM weights/biases,
    kif WRAP datalane quantizers, EBOPs with beta0."""

    def __init__(self, dims=(16, 64, 32, 32, 5), beta0=1e-5, seed=0, batch_shape_tail=None):
        g = torch.Generator().manual_seed(seed)
        self.layers = []
        for n, (din, dout) in enumerate(zip(dims[:-1], dims[1:])):
            kernel = glorot_uniform((din, dout), g)
            bias = torch.zeros(dout)
            iq = default_quantizer('datalane', (None, din), q_type='kif', overflow_mode='WRAP')
            kq = default_quantizer('weight', (din, dout), q_type='kbi', overflow_mode='SAT_SYM')
            bq = default_quantizer('bias', (dout,), q_type='kbi', overflow_mode='SAT_SYM')
            act = 'relu' if n < len(dims) - 2 else None
            self.layers.append(RefQDense(kernel, bias, iq, kq, bq, activation=act, beta0=beta0))

    def forward(self, x, training=True):
        for layer in self.layers:
            x = layer(x, training=training)
        return x

    def trainable_variables(self):
        out = []
        for layer in self.layers:
            out += layer.trainable_variables()
        return out

    def loss(self, x, labels, training=True):
        logits = self.forward(x, training=training)
        loss = F.cross_entropy(logits, labels)
        for layer in self.layers:
            loss = loss + layer.extra_loss()
        return loss, logits

    def train_step(self, x, labels, lr=0.01):
        variables = self.trainable_variables()
        for v in variables:
            v.grad = None
        loss, logits = self.loss(x, labels, training=True)
        loss.backward()
        with torch.no_grad():
            for v in variables:
                if v.grad is not None:
                    v.sub_(lr * v.grad)
        for layer in self.layers:
            layer.apply_constraints()
        return loss.detach(), logits.detach()
