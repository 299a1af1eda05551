from ..quantizer import Quantizer
from .core import QDense, QEinsumDense, QLayerBase, QLayerBaseMultiInputs, QLayerBaseSingleInput

__all__ = ['Quantizer', 'QDense', 'QEinsumDense', 'QLayerBase', 'QLayerBaseSingleInput', 'QLayerBaseMultiInputs']
