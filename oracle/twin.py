"""Build the CPU oracle's twin of a product layer: same configuration, same variable values."""

import torch

from . import hgq_ref as ref


def _constraint(c):
    if c is None:
        return None
    from hgq2_amd.constraints import Constant, Max, Min, MinMax

    if isinstance(c, MinMax):
        return ('minmax', c.min_value, c.max_value)
    if isinstance(c, Constant):
        return ('constant', c.value)
    if isinstance(c, Min):
        return ('min', c.min_value)
    if isinstance(c, Max):
        return ('max', c.max_value)
    raise TypeError(c)


def _reg(r):
    return None if r is None else r.l1


PAIRS = []  # (product internal quantizer, oracle internal quantizer) of every twin built since the list was cleared


def ref_quantizer(q):
    """hgq2_amd.quantizer.Quantizer -> oracle RefQuantizer with copied variables."""
    if q is None:
        return None
    inner = q.quantizer
    if q.config.q_type == 'dummy':
        return ref.RefQuantizer(ref.RefDummyQuantizer(), q.scaler, q.affine, q.qnoise_factor)
    cfg = q.config.config
    shape = tuple(inner._i.shape)
    kw = dict(round_mode=inner.round_mode, overflow_mode=inner.overflow_mode, ic=_constraint(cfg.get('ic')),
              ir=_reg(cfg.get('ir')), i_decay_speed=cfg['i_decay_speed'], heterogeneous_axis=tuple(range(len(shape))),
              is_weight=cfg['is_weight'], trainable=cfg['trainable'], seed=getattr(inner, '_seed', 0))
    if q.config.q_type == 'kif':
        kw.update(fc=_constraint(cfg.get('fc')), fr=_reg(cfg.get('fr')))
    else:
        kw.update(bc=_constraint(cfg.get('bc')), br=_reg(cfg.get('br')))
    # the oracle quantizer is built on the bit-width shape itself and told which axes broadcast
    r = ref.RefFixedPointQuantizer(q.config.q_type, shape, **kw)
    r.bw_mapper = ref.BitwidthMapper(heterogeneous_axis=tuple(inner.bw_mapper.heterogeneous_axis))
    r.bw_mapper.homogeneous_axis = tuple(inner.bw_mapper.homogeneous_axis)
    with torch.no_grad():
        r._k.copy_(inner._k.detach().cpu())
        r._i.copy_(inner._i.detach().cpu())
        if q.config.q_type == 'kif':
            r._f.copy_(inner._f.detach().cpu())
        else:
            r._b.copy_(inner._b.detach().cpu())
    if r.seed_gen is not None:  # both sides continue from the same position of the same stream
        r.seed_gen.seed, r.seed_gen.offset = inner._seed_gen.seed, inner._seed_gen.offset
    PAIRS.append((inner, r))
    return ref.RefQuantizer(r, q.scaler, q.affine, q.qnoise_factor)


def _beta(layer):
    return float(layer._beta) if layer._beta is not None else 0.0


def _iq(layer):
    return ref_quantizer(layer.iq) if layer.enable_iq else None


def _oq(layer):
    return ref_quantizer(layer.oq) if layer.enable_oq else None


def ref_dense(layer):
    return ref.RefQDense(layer._kernel.detach().cpu(), None if layer.bias is None else layer.bias.detach().cpu(),
                         _iq(layer), ref_quantizer(layer.kq), ref_quantizer(layer.bq),
                         activation=None if layer._act_name == 'linear' else layer._act_name, beta0=_beta(layer),
                         enable_ebops=layer.enable_ebops, parallelization_factor=layer.parallelization_factor,
                         n_parallel=layer.n_parallel, oq=_oq(layer))


def ref_einsum_dense(layer, input_shape, cls=None, **extra):
    cls = cls or ref.RefQEinsumDense
    return cls(layer.equation, layer._kernel.detach().cpu(), None if layer.bias is None else layer.bias.detach().cpu(),
               _iq(layer), ref_quantizer(layer.kq), ref_quantizer(layer.bq), tuple(input_shape),
               tuple(layer.full_output_shape[1:]), activation=None if layer._act_name == 'linear' else layer._act_name,
               beta0=_beta(layer), enable_ebops=layer.enable_ebops, parallelization_factor=layer.parallelization_factor,
               oq=_oq(layer), **extra)


def ref_einsum_dense_bn(layer, input_shape):
    return ref_einsum_dense(layer, input_shape, cls=ref.RefQEinsumDenseBatchnorm,
                            gamma=layer.bn_gamma.detach().cpu() if layer.scale else None,
                            moving_mean=layer.moving_mean.detach().cpu(),
                            moving_variance=layer.moving_variance.detach().cpu(), normalize_axes=layer.normalize_axes,
                            momentum=layer.momentum)


def ref_batchnorm(layer):
    return ref.RefQBatchNormalization(layer.axis, layer.bn_gamma.detach().cpu() if layer.scale else None,
                                      layer.bn_beta.detach().cpu() if layer.center else None, layer.moving_mean.detach().cpu(),
                                      layer.moving_variance.detach().cpu(), _iq(layer), ref_quantizer(layer.kq), ref_quantizer(layer.bq),
                                      momentum=layer.momentum, epsilon=layer.epsilon, beta0=_beta(layer),
                                      enable_ebops=layer.enable_ebops)


def ref_lut(layer, fn):
    return ref.RefQUnaryFunctionLUT(fn, _iq(layer), _oq(layer), beta0=_beta(layer), enable_ebops=layer.enable_ebops)


def ref_softmax(layer):
    scaler = layer.input_scaler
    sign = -1.0 if layer.stable else 1.0
    exp = ref_lut(layer.exp_table, lambda x: torch.exp(sign * x * scaler))
    inv = ref_lut(layer.inv_table, lambda x: 1.0 / (x + ref.EPSILON))
    return ref.RefQSoftmax(layer.axes, exp, inv, _oq(layer), iq=_iq(layer), input_scaler=scaler, beta0=_beta(layer),
                           enable_ebops=layer.enable_ebops, parallelization_factor=layer.parallelization_factor,
                           stable=layer.stable)


def ref_mha(layer, query_shape, value_shape=None, key_shape=None):
    value_shape = query_shape if value_shape is None else value_shape
    key_shape = value_shape if key_shape is None else key_shape
    N = layer._num_heads
    qd = ref_einsum_dense(layer._query_dense, query_shape)
    kd = ref_einsum_dense(layer._key_dense, key_shape)
    vd = ref_einsum_dense(layer._value_dense, value_shape)
    od = ref_einsum_dense(layer._output_dense, tuple(query_shape[:-1]) + (N, layer._value_dim))
    # fused input quantizers are one shared object in the product; share the twin as well
    for d, own in ((qd, layer._query_dense), (kd, layer._key_dense)):
        if own.enable_iq and own._iq is layer._value_dense._iq:
            orphan = d.iq.quantizer
            d.iq = vd.iq
            PAIRS[:] = [pair for pair in PAIRS if pair[1] is not orphan]  # the twin that was built for it is never called
    return ref.RefQMultiHeadAttention(qd, kd, vd, od, ref_softmax(layer._softmax), beta0=_beta(layer),
                                      enable_ebops=layer.enable_ebops, parallelization_factor=layer.parallelization_factor)


def ref_conv2d(layer):
    return ref.RefQConv2D(layer._kernel.detach().cpu(), None if layer.bias is None else layer.bias.detach().cpu(),
                          _iq(layer), ref_quantizer(layer.kq), ref_quantizer(layer.bq), strides=layer.strides,
                          padding=layer.padding, activation=None if layer._act_name == 'linear' else layer._act_name,
                          beta0=_beta(layer), enable_ebops=layer.enable_ebops,
                          parallelization_factor=layer.parallelization_factor, n_parallel=layer.n_parallel, oq=_oq(layer))


def quantizer_pairs(ref_layer_quantizers, prod_quantizers):
    return list(zip(ref_layer_quantizers, prod_quantizers))


def ref_pooling2d(layer):
    return ref.RefQPooling2D(layer._mode, layer.pool_size, layer.strides, layer.padding, _iq(layer), oq=_oq(layer),
                             beta0=_beta(layer), enable_ebops=layer.enable_ebops,
                             parallelization_factor=layer.parallelization_factor, n_parallel=layer.n_parallel)
