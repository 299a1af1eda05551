"""The reference's import paths resolve to this build's modules (``hgq`` package at the repository root), and the
README example of the reference constructs unchanged.  CPU only: nothing here launches a kernel."""

import importlib

import pytest


def test_reference_module_paths_resolve_to_the_same_objects():
    import hgq
    import hgq2_amd

    assert set(hgq.__all__) >= {'config', 'layers', 'quantizer', 'utils'}  # reference src/hgq/__init__.py:26-29
    for path, names in {
        'hgq.layers': ['QDense', 'QEinsumDense', 'QEinsumDenseBatchnorm', 'QConv2D', 'QSoftmax', 'QMultiHeadAttention',
                       'QUnaryFunctionLUT', 'QBatchNormalization', 'QMaxPool2D', 'QAvgPool2D', 'QMaxPooling2D',
                       'QGlobalAvgPool1D', 'Quantizer'],
        'hgq.layers.core': ['QDense', 'QEinsumDense', 'QLayerBase'],
        'hgq.layers.core.dense': ['QDense'],
        'hgq.layers.core.einsum_dense': ['QEinsumDense'],
        'hgq.layers.core.base': ['QLayerBase', 'QLayerBaseSingleInput', 'QLayerBaseMultiInputs'],
        'hgq.layers.conv': ['QConv2D'],
        'hgq.layers.softmax': ['QSoftmax'],
        'hgq.layers.activation': ['QUnaryFunctionLUT'],
        'hgq.layers.einsum_dense_batchnorm': ['QEinsumDenseBatchnorm'],
        'hgq.layers.attn.mha': ['QMultiHeadAttention'],
        'hgq.layers.batch_normalization': ['QBatchNormalization'],
        'hgq.layers.pooling': ['QMaxPooling2D', 'QAveragePooling2D'],
        'hgq.quantizer': ['Quantizer', 'QuantizerConfig'],
        'hgq.quantizer.config': ['QuantizerConfig', 'QuantizerConfigScope', 'default_configs'],
        'hgq.quantizer.quantizer': ['Quantizer'],
        'hgq.quantizer.internal': ['FixedPointQuantizerKBI', 'FixedPointQuantizerKIF', 'DummyQuantizer'],
        'hgq.quantizer.internal.fixed_point_quantizer': ['FixedPointQuantizerBase', 'FixedPointQuantizerKBI', 'FixedPointQuantizerKIF'],
        'hgq.quantizer.internal.base': ['DefaultBitwidthMapper', 'TrainableQuantizerBase', 'round_conv'],
        'hgq.config': ['LayerConfigScope', 'QuantizerConfigScope', 'QuantizerConfig', 'global_config', 'default_configs'],
        'hgq.config.layer': ['LayerConfigScope', 'global_config'],
        'hgq.config.quantizer': ['QuantizerConfig', 'QuantizerConfigScope', 'default_configs'],
        'hgq.constraints': ['MinMax', 'Min', 'Max', 'Constant'],
        'hgq.regularizers': ['MonoL1'],
        'hgq.utils': ['trace_minmax'],
        'hgq.utils.minmax_trace': ['trace_minmax'],
        'hgq.utils.sugar': ['BetaScheduler', 'PieceWiseSchedule', 'BetaPID', 'FreeEBOPs'],
        'hgq.utils.sugar.beta_scheduler': ['BetaScheduler', 'PieceWiseSchedule'],
        'hgq.utils.sugar.beta_pid': ['BetaPID'],
        'hgq.utils.sugar.ebops': ['FreeEBOPs'],
    }.items():
        mod = importlib.import_module(path)
        for name in names:
            assert hasattr(mod, name), f'{path}.{name}'
    assert hgq.layers.QDense is hgq2_amd.layers.QDense
    assert hgq.config.QuantizerConfigScope is hgq2_amd.quantizer.config.QuantizerConfigScope
    from hgq.quantizer.internal.fixed_point_quantizer import FixedPointQuantizerKIF

    assert FixedPointQuantizerKIF is hgq2_amd.quantizer.internal.FixedPointQuantizerKIF


def test_readme_example_constructs_with_only_the_host_import_swapped():
    """Reference README.md:57-67, verbatim but for the first import."""
    import hgq2_amd.host as keras
    from hgq.config import LayerConfigScope, QuantizerConfigScope
    from hgq.layers import QConv2D, QDense
    from hgq2_amd.core import set_default_device

    set_default_device('cpu')
    try:
        with (
            QuantizerConfigScope(place='all', default_q_type='kbi', overflow_mode='SAT_SYM'),
            QuantizerConfigScope(place='datalane', default_q_type='kif', overflow_mode='WRAP'),
            LayerConfigScope(enable_ebops=True, beta0=1e-5),
        ):
            model = keras.Sequential([
                QConv2D(32, (3, 3), activation='relu'),
                keras.layers.MaxPooling2D((2, 2)),
                keras.layers.Flatten(),
                QDense(10)
            ])
        conv, pool, flat, dense = model.layers
        shape = (None, 28, 28, 1)
        conv.build(shape)
        shape = pool.compute_output_shape(conv.compute_output_shape(shape))
        assert shape == (None, 13, 13, 32)
        dense.build(flat.compute_output_shape(shape))
    finally:
        set_default_device(None)
    from hgq.quantizer.internal import FixedPointQuantizerKBI, FixedPointQuantizerKIF

    assert isinstance(conv.iq.quantizer, FixedPointQuantizerKIF) and conv.iq.quantizer.overflow_mode == 'WRAP'
    assert isinstance(conv.kq.quantizer, FixedPointQuantizerKBI) and conv.kq.quantizer.overflow_mode == 'SAT_SYM'
    assert tuple(conv.iq.quantizer._i.shape) == (1, 28, 28, 1) and tuple(conv.kq.quantizer._b.shape) == (3, 3, 1, 32)
    assert tuple(dense.kq.quantizer._b.shape) == (13 * 13 * 32, 10)
    assert float(conv._beta) == pytest.approx(1e-5) and conv.enable_ebops


def test_operators_refuse_cpu_tensors():
    """There is no CPU implementation behind the namespace: a quantizer call on a CPU tensor raises."""
    import torch

    from hgq.quantizer import Quantizer, QuantizerConfig

    q = Quantizer(QuantizerConfig('kif', 'datalane'))
    with pytest.raises((ValueError, RuntimeError)):
        q(torch.zeros(4, 3), training=True)
