from ..quantizer import Quantizer
from .activation import QUnaryFunctionLUT
from .attn import QMultiHeadAttention
from .conv import QConv2D
from .core import QDense, QEinsumDense, QLayerBase, QLayerBaseMultiInputs, QLayerBaseSingleInput
from .einsum_dense_batchnorm import QEinsumDenseBatchnorm
from .softmax import QSoftmax

__all__ = ['Quantizer', 'QDense', 'QEinsumDense', 'QEinsumDenseBatchnorm', 'QConv2D', 'QSoftmax', 'QUnaryFunctionLUT',
           'QMultiHeadAttention', 'QLayerBase', 'QLayerBaseSingleInput', 'QLayerBaseMultiInputs']
