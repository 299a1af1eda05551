"""Scoped layer defaults (reference src/hgq/config/layer.py:6-41)."""

from __future__ import annotations

global_config = dict(
    beta0=1e-5,
    enable_ebops=True,
    enable_oq=False,
    enable_iq=True,
    enable_sq=True,
)


class LayerConfigScope:
    """``with LayerConfigScope(enable_ebops=True, beta0=1e-5): ...`` overrides the defaults
    read by layers at construction time."""

    def __init__(self, **kwargs):
        self._override = kwargs

    def __enter__(self):
        self._tmp = global_config.copy()
        for k, v in self._override.items():
            global_config[k] = v

    def __exit__(self, exc_type, exc_val, exc_tb):
        for k in self._override:
            global_config.pop(k, None)
        global_config.update(self._tmp)
