from ..quantizer import Quantizer
from .activation import QUnaryFunctionLUT
from .attn import QMultiHeadAttention
from .batch_normalization import QBatchNormalization
from .conv import QConv2D
from .core import QDense, QEinsumDense, QLayerBase, QLayerBaseMultiInputs, QLayerBaseSingleInput
from .einsum_dense_batchnorm import QEinsumDenseBatchnorm
from .pooling import (QAveragePooling2D, QGlobalAveragePooling1D, QGlobalAveragePooling2D, QGlobalMaxPooling1D,
                      QGlobalMaxPooling2D, QMaxPooling2D)
from .softmax import QSoftmax

# short names of the reference (src/hgq/layers/__init__.py:9-44)
QMaxPool2D, QAvgPool2D = QMaxPooling2D, QAveragePooling2D
QGlobalAvgPool1D, QGlobalAvgPool2D = QGlobalAveragePooling1D, QGlobalAveragePooling2D
QGlobalMaxPool1D, QGlobalMaxPool2D = QGlobalMaxPooling1D, QGlobalMaxPooling2D

__all__ = ['Quantizer', 'QDense', 'QEinsumDense', 'QEinsumDenseBatchnorm', 'QBatchNormalization', 'QConv2D', 'QSoftmax', 'QUnaryFunctionLUT',
           'QMultiHeadAttention', 'QMaxPooling2D', 'QAveragePooling2D', 'QGlobalAveragePooling1D', 'QGlobalAveragePooling2D',
           'QGlobalMaxPooling1D', 'QGlobalMaxPooling2D', 'QMaxPool2D', 'QAvgPool2D', 'QGlobalAvgPool1D', 'QGlobalAvgPool2D',
           'QGlobalMaxPool1D', 'QGlobalMaxPool2D', 'QLayerBase', 'QLayerBaseSingleInput', 'QLayerBaseMultiInputs']
