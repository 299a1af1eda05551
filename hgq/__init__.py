"""The reference's import paths, served by ``hgq2_amd``.

``import hgq`` registers every module of ``hgq2_amd`` under the name the reference gives it (``hgq.layers``,
``hgq.layers.core.dense``, ``hgq.quantizer.internal.fixed_point_quantizer``, ``hgq.config``, ``hgq.utils.sugar``,
``hgq.constraints``, ``hgq.regularizers`` ...), so user code written against the reference package
(reference src/hgq/__init__.py:26-29, README.md:57-67) imports unchanged.  The objects are the same objects:
``hgq.layers.QDense is hgq2_amd.layers.QDense``.  Nothing is implemented here.
"""

import importlib
import importlib.util
import pkgutil
import sys

import hgq2_amd as _impl

# reference module paths whose contents live in a differently named module here
_RENAMED = {
    'hgq.config.quantizer': 'hgq2_amd.quantizer.config',                   # reference src/hgq/config/quantizer.py
    'hgq.utils.sugar.beta_scheduler': 'hgq2_amd.utils.sugar.callbacks',    # reference src/hgq/utils/sugar/beta_scheduler.py
    'hgq.utils.sugar.beta_pid': 'hgq2_amd.utils.sugar.callbacks',          # reference src/hgq/utils/sugar/beta_pid.py
    'hgq.utils.sugar.ebops': 'hgq2_amd.utils.sugar.callbacks',             # reference src/hgq/utils/sugar/ebops.py
}


def _register():
    for info in pkgutil.walk_packages(_impl.__path__, _impl.__name__ + '.'):
        spec = importlib.util.find_spec(info.name)
        if spec is None or not (spec.origin or '').endswith('.py'):
            continue  # the built HIP library sits in the package directory and is not a Python module
        mod = importlib.import_module(info.name)
        sys.modules[__name__ + info.name[len(_impl.__name__):]] = mod
    for alias, target in _RENAMED.items():
        mod = sys.modules[alias] = importlib.import_module(target)
        parent, leaf = alias.rsplit('.', 1)
        setattr(sys.modules[parent], leaf, mod)  # `import a.b.c as m` reads c as an attribute of a.b


_register()

from hgq2_amd import config, constraints, layers, quantizer, regularizers, utils  # noqa: E402,F401

__version__ = _impl.__version__
__all__ = ['config', 'layers', 'quantizer', 'utils', 'constraints', 'regularizers']
