"""hgq2_amd: the HGQ2 quantized-training hot path on MI355X.

The public surface mirrors the reference package layout (``hgq.config``, ``hgq.layers``,
``hgq.quantizer``, ``hgq.constraints``, ``hgq.regularizers``); the arithmetic runs in hand-written
HIP kernels (``libhgq_hip.so``) reached through ``torch.library`` operators.
"""

from . import config, constraints, layers, quantizer, regularizers  # noqa: F401

__version__ = '0.1.0'
__all__ = ['config', 'layers', 'quantizer', 'constraints', 'regularizers']
