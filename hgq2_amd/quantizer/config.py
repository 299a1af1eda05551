"""Quantizer configuration: defaults per (quantizer type, place), ``QuantizerConfig`` and the
``QuantizerConfigScope`` context manager.

Mirrors the interface and default values of reference src/hgq/quantizer/config.py:21-26 (default
types), :75-220 (default configs), :240-548 (QuantizerConfig), :550-638 (scope), :641-720 (hard
tanh / sigmoid sugar).  The minifloat quantizer type keeps its configuration keys so scopes behave
the same, but constructing it raises: it is outside the fixed-point hot path.
"""

from __future__ import annotations

from collections.abc import Mapping

from ..constraints import Constant, Min, MinMax
from ..regularizers import MonoL1

default_q_type = {'weight': 'kbi', 'datalane': 'kif', 'bias': 'kbi', 'table': 'kbi'}

_COMMON_KEYS = ('homogeneous_axis', 'heterogeneous_axis', 'bw_mapper', 'trainable', 'is_weight')


def _kbi(place_kw):
    base = dict(k0=True, b0=8, i0=2, round_mode='RND', overflow_mode='SAT_SYM', bc=MinMax(0, 23), ic=None,
                br=MonoL1(1e-8), ir=None, i_decay_speed=float('inf'), homogeneous_axis=(), heterogeneous_axis=None,
                bw_mapper=None, trainable=True, is_weight=True)
    base.update(place_kw)
    return base


def _kif(place_kw):
    base = dict(k0=True, i0=2, f0=6, round_mode='RND', overflow_mode='SAT_SYM', ic=MinMax(-23, 23), ir=MonoL1(1e-8),
                fc=MinMax(-24, 24), fr=MonoL1(1e-8), i_decay_speed=float('inf'), homogeneous_axis=(),
                heterogeneous_axis=None, bw_mapper=None, trainable=True, is_weight=True)
    base.update(place_kw)
    return base


def _float(place_kw):
    base = dict(m0=2, e0=4, e00=0, mc=MinMax(-1, 8), ec=MinMax(0, 4), e0c=MinMax(-16, 16), mr=MonoL1(1e-8),
                er=MonoL1(1e-8), e0r=None, homogeneous_axis=(), heterogeneous_axis=None, bw_mapper=None, trainable=True,
                is_weight=True)
    base.update(place_kw)
    return base


_datalane = dict(overflow_mode='WRAP', i_decay_speed=0.01, homogeneous_axis=(0,), is_weight=False)
_table = dict(homogeneous_axis=None, heterogeneous_axis=(), is_weight=False)
_bias = dict(overflow_mode='WRAP', i_decay_speed=0.01, homogeneous_axis=(), is_weight=False)

default_configs: dict[tuple[str, str], dict] = {
    ('kbi', 'weight'): _kbi({}),
    ('kbi', 'bias'): _kbi(dict(_bias, bc=MinMax(0, 24))),
    ('kbi', 'table'): _kbi(_table),
    ('kbi', 'datalane'): _kbi(dict(_datalane, bc=MinMax(0, 24))),
    ('kif', 'weight'): _kif({}),
    ('kif', 'bias'): _kif(_bias),
    ('kif', 'table'): _kif(_table),
    ('kif', 'datalane'): _kif(_datalane),
    ('float', 'weight'): _float({}),
    ('float', 'bias'): _float(dict(homogeneous_axis=(), heterogeneous_axis=None, is_weight=False)),
    ('float', 'table'): _float(_table),
    ('float', 'datalane'): _float(dict(homogeneous_axis=None, heterogeneous_axis=(), is_weight=False)),
}

all_quantizer_keys = {k for v in default_configs.values() for k in v.keys()} | {
    'q_type', 'place', 'scaler', 'affine', 'qnoise_factor',
}


def all_quantizer_types():
    return {k[0] for k in default_configs}


def all_places():
    return {k[1] for k in default_configs}


def _normalise_axes(kwargs):
    assert kwargs.get('homogeneous_axis') is None or kwargs.get('heterogeneous_axis') is None, (
        'homogeneous_axis and heterogeneous_axis are mutually exclusive. Set only one of them.'
    )
    if kwargs.get('homogeneous_axis') is not None:
        kwargs['heterogeneous_axis'] = None
    if kwargs.get('heterogeneous_axis') is not None:
        kwargs['homogeneous_axis'] = None


class QuantizerConfig(Mapping):
    """Universal quantizer config; ``q_type`` in {'kbi', 'kif', 'float', 'dummy', 'default'},
    ``place`` in {'weight', 'datalane', 'bias', 'table'}; remaining keyword arguments override the
    default config of that (type, place)."""

    def __init__(self, q_type='default', place='datalane', scaler=None, affine=None, qnoise_factor=None, **kwargs):
        place = place.lower()
        q_type = q_type.lower()
        if q_type == 'default':
            q_type = default_q_type[place]
        if q_type != 'dummy':
            assert (q_type, place) in default_configs, f'Default config for ({q_type}, {place}) not found.'
        self.place = place
        self.q_type = q_type
        self.scaler = None
        self.qnoise_factor = None
        self.affine = None
        if scaler is not None:
            assert scaler != 0, 'scaler must not be 0.'
            self.scaler = float(scaler)
        if affine is not None:
            assert len(affine) == 2, 'affine must be a tuple of (scale, shift).'
            assert affine[0] != 0, 'affine scale must not be 0.'
            self.affine = (float(affine[0]), float(affine[1]))
        if qnoise_factor is not None:
            assert 0 <= qnoise_factor <= 1, 'qnoise_factor must be between 0 and 1.'
            self.qnoise_factor = float(qnoise_factor)
        if q_type == 'dummy':
            self.config = {}
            return
        _normalise_axes(kwargs)
        self.config = default_configs[(q_type, place)].copy()
        for k, v in kwargs.items():
            if k not in self.config:
                raise ValueError(f'{k} is not a valid parameter for {q_type} quantizer config.')
            self.config[k] = v

    def __getitem__(self, key):
        return self.config[key]

    def __iter__(self):
        return iter(self.config)

    def __len__(self):
        return len(self.config)

    def __bool__(self):
        return True

    def get_config(self):
        return {'q_type': self.q_type, 'place': self.place, 'scaler': self.scaler, 'qnoise_factor': self.qnoise_factor,
                'affine': self.affine, **self.config}

    @classmethod
    def from_config(cls, config):
        return cls(**config)

    def copy(self):
        new = QuantizerConfig.__new__(type(self))
        new.__dict__.update(self.__dict__)
        new.config = self.config.copy()
        return new

    def get_quantizer(self):
        from .internal import DummyQuantizer, FixedPointQuantizerKBI, FixedPointQuantizerKIF

        if self.q_type == 'kif':
            return FixedPointQuantizerKIF(**self)
        if self.q_type == 'kbi':
            return FixedPointQuantizerKBI(**self)
        if self.q_type == 'dummy':
            return DummyQuantizer()
        if self.q_type == 'float':
            raise NotImplementedError('the minifloat quantizer is outside the fixed-point hot path of this build')
        raise ValueError(f'Unknown quantizer type: {self.q_type}')


class QuantizerConfigScope:
    """Override default quantizer configs (and optionally the default quantizer type) within a
    context.  Only keys that exist in a given default config are overridden."""

    def __init__(self, q_type='all', place='all', default_q_type=None, **kwargs):
        if q_type == 'all':
            q_type = all_quantizer_types()
        if place == 'all':
            place = all_places()
        q_type = (q_type,) if isinstance(q_type, str) else q_type
        place = (place,) if isinstance(place, str) else place
        self.q_types = {t.lower() for t in q_type}
        self.places = {p.lower() for p in place}
        for t in self.q_types:
            for p in self.places:
                assert (t, p) in default_configs, f'Default config for ({t}, {p}) not found.'
        _normalise_axes(kwargs)
        i, f, b = kwargs.get('i0'), kwargs.get('f0'), kwargs.get('b0')
        if sum(v is not None for v in (i, f, b)) == 2:
            if i is None:
                kwargs['i0'] = b - f
            if f is None:
                kwargs['f0'] = b - i
            if b is None:
                kwargs['b0'] = i + f
        for k in kwargs:
            if k not in all_quantizer_keys:
                raise ValueError(f'{k} is not a valid parameter for any known quantizer configs.')
        self.kwargs = kwargs
        self.default_q_type = default_q_type
        self._saved = {}
        self._saved_q_type = None

    def __enter__(self):
        for key, conf in default_configs.items():
            if key[0] in self.q_types and key[1] in self.places:
                self._saved[key] = conf.copy()
                for k, v in self.kwargs.items():
                    if k in conf:
                        conf[k] = v
        if self.default_q_type is not None:
            self._saved_q_type = default_q_type.copy()
            for place in self.places:
                default_q_type[place] = self.default_q_type

    def __exit__(self, exc_type, exc_value, traceback):
        if self._saved_q_type is not None:
            default_q_type.clear()
            default_q_type.update(self._saved_q_type)
            self._saved_q_type = None
        for key, conf in self._saved.items():
            default_configs[key].update(conf)
        self._saved.clear()

    def override(self):
        """Make the override permanent."""
        self.__enter__()
        self._saved.clear()


class HardTanhConfig(QuantizerConfig):
    """A [-1, 1) saturating quantizer: ``q_type='kif', k0=1, i0=0, ic=Constant(0)``."""

    def __init__(self, q_type='kif', place='datalane', symmetric=False, **kwargs):
        assert not any(k in kwargs for k in ('k0', 'ic', 'affine', 'overflow_mode')), (
            'k0, ic, affine, overflow_mode must not be set for HardTanhConfig.'
        )
        kwargs.pop('i0', None)
        super().__init__(q_type=q_type, place=place, k0=1, ic=Constant(0), i0=0,
                         overflow_mode='SAT_SYM' if symmetric else 'SAT', affine=None, **kwargs)


class HardSigmoidConfig(QuantizerConfig):
    """A [0, 1) saturating quantizer: ``k0=1, i0=1, ic=Constant(1), affine=(0.25, 0.5)``."""

    def __init__(self, q_type='kif', place='datalane', **kwargs):
        assert not any(k in kwargs for k in ('k0', 'ic', 'affine', 'overflow_mode')), (
            'k0, ic, affine, overflow_mode must not be set for HardSigmoidConfig.'
        )
        kwargs.pop('i0', None)
        super().__init__(q_type=q_type, place=place, k0=1, ic=Constant(1), i0=1, overflow_mode='SAT',
                         affine=(0.25, 0.5), **kwargs)


__all__ = ['QuantizerConfig', 'QuantizerConfigScope', 'HardTanhConfig', 'HardSigmoidConfig', 'default_configs',
           'default_q_type', 'all_quantizer_keys', 'Min']
