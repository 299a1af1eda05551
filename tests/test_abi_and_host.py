"""CPU-side checks: the C-ABI library loads and exports every symbol the header declares, the
ctypes table matches the header, and the host logic (config scopes, bit-width layouts, einsum
analysis) behaves as the reference's does.  No compute call is made here."""

import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, 'include', 'hgq_hip.h')).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(hgq_[a-z0-9_]+)\s*\(', text)))


def test_library_exports_every_declared_symbol():
    from hgq2_amd import _lib

    lib = _lib.load()
    names = _declared()
    assert len(names) >= 12
    for n in names:
        assert hasattr(lib, n), f'{n} is declared in include/hgq_hip.h but not exported'
        assert n in _lib.SIGNATURES, f'{n} has no ctypes signature'
    assert sorted(_lib.SIGNATURES) == names
    assert lib.hgq_version() >= 1


def test_mode_bits_match_header():
    from hgq2_amd import _lib

    text = open(os.path.join(ROOT, 'include', 'hgq_hip.h')).read()
    for name in ('TRAINING', 'KBI', 'ROUND_PARAMS', 'K_U8', 'SYMMETRIC', 'TRACING', 'TRACK_INPUT'):
        shift = int(re.search(rf'#define HGQ_MODE_{name} \(1 << (\d+)\)', text).group(1))
        assert getattr(_lib, f'MODE_{name}') == 1 << shift
    assert _lib.mode_bits('RND', 'SAT_SYM', training=True, kbi=True) == 1 | (2 << 4) | (1 << 8) | (1 << 9)
    with pytest.raises(ValueError):
        _lib.mode_bits('RND', 'NOPE')


def test_ops_refuse_cpu_tensors():
    from hgq2_amd import _lib, ops

    x = torch.zeros(8)
    with pytest.raises(ValueError, match='GPU'):
        ops.quantize(x, x, x, x, _lib.mode_bits('RND', 'WRAP'))


def test_missing_library_fails_loudly(monkeypatch):
    from hgq2_amd import _lib

    monkeypatch.setattr(_lib, '_lib', None)
    monkeypatch.setattr(_lib, 'LIB_PATH', '/nonexistent/libhgq_hip.so')
    with pytest.raises(_lib.HGQLibraryError, match='no CPU fallback'):
        _lib.load()


def test_quantizer_config_scopes_follow_reference_semantics():
    from hgq2_amd.config import LayerConfigScope, QuantizerConfig, QuantizerConfigScope, global_config
    from hgq2_amd.quantizer.config import default_configs, default_q_type

    before = {k: dict(v) for k, v in default_configs.items()}
    with QuantizerConfigScope(place='all', default_q_type='kbi', overflow_mode='SAT_SYM'):
        with QuantizerConfigScope(place='datalane', default_q_type='kif', overflow_mode='WRAP'):
            assert QuantizerConfig('default', 'datalane').q_type == 'kif'
            assert QuantizerConfig('default', 'datalane')['overflow_mode'] == 'WRAP'
            assert QuantizerConfig('default', 'bias')['overflow_mode'] == 'SAT_SYM'
            assert QuantizerConfig('default', 'weight').q_type == 'kbi'
            assert 'overflow_mode' not in default_configs[('float', 'weight')]
        assert default_q_type['datalane'] == 'kbi'
    assert {k: dict(v) for k, v in default_configs.items()} == before
    assert default_q_type == {'weight': 'kbi', 'datalane': 'kif', 'bias': 'kbi', 'table': 'kbi'}
    # explicit kwargs beat the scope; unknown keys are rejected; two of (i0, f0, b0) imply the third
    with QuantizerConfigScope(place='datalane', overflow_mode='WRAP'):
        assert QuantizerConfig(place='datalane', overflow_mode='SAT')['overflow_mode'] == 'SAT'
    with pytest.raises(ValueError):
        QuantizerConfig('kif', 'datalane', b0=3)
    s = QuantizerConfigScope(i0=2, b0=6)
    assert s.kwargs['f0'] == 4
    with LayerConfigScope(beta0=0.5, enable_ebops=False):
        assert global_config['beta0'] == 0.5 and global_config['enable_ebops'] is False
    assert global_config['beta0'] == 1e-5 and global_config['enable_ebops'] is True
    d = default_configs[('kif', 'datalane')]
    assert (d['k0'], d['i0'], d['f0'], d['i_decay_speed'], d['homogeneous_axis']) == (True, 2, 6, 0.01, (0,))
    w = default_configs[('kbi', 'weight')]
    assert (w['b0'], w['i0'], w['overflow_mode'], w['bc'].max_value, w['is_weight']) == (8, 2, 'SAT_SYM', 23.0, True)


def test_bitwidth_layouts():
    from hgq2_amd.quantizer.internal import DefaultBitwidthMapper
    from hgq2_amd.quantizer.internal.base import bw_layout

    m = DefaultBitwidthMapper(None, (0,))
    assert m.inference_weight_shape((None, 28, 28, 1)) == (1, 28, 28, 1)
    m = DefaultBitwidthMapper((), None)
    assert m.inference_weight_shape((None, 4, 64, 64)) == (1, 1, 1, 1)
    assert bw_layout((1, 16), (4096, 16)) == (16, 1)
    assert bw_layout((16, 64), (16, 64)) == (1024, 1)
    assert bw_layout((1, 1, 1), (33, 5, 8)) == (1, 1)
    assert bw_layout((1, 6, 1), (50, 6, 4)) == (6, 4)
    assert bw_layout((1, 4, 64, 64), (2048, 4, 64, 64)) == (16384, 1)
    assert bw_layout((3, 1, 5), (3, 4, 5)) is None


def test_einsum_analysis():
    from hgq2_amd.layers.core.einsum_dense import _einsum_free0_size, analyze_einsum_string, gemm_form

    assert analyze_einsum_string('abc,cde->abde', 'de', (None, 64, 64), (64, 4, 16)) == ((64, 4, 16), (4, 16), (None, 64, 4, 16))
    assert analyze_einsum_string('abcd,cde->abe', 'e', (None, 64, 4, 16), (64, 64)) == ((4, 16, 64), (64,), (None, 64, 64))
    assert analyze_einsum_string('Babc,bcd->Babd', 'ad', (None, 3, 4, 5), (3, 4, 2))[1] == (3, 1, 2)
    assert gemm_form('bpf,fh->bph') == (1, 1) and gemm_form('abc,cde->abde') == (1, 2)
    assert gemm_form('abcd,cde->abe') == (2, 1) and gemm_form('Bij,ijk->Bik') is None
    assert _einsum_free0_size('bpf,fh->bph', (None, 64, 16)) == 64
    assert _einsum_free0_size('Bij,ijk->Bik', (None, 3, 4)) == 1


def test_constraints_and_regularizers():
    from hgq2_amd.constraints import Constant, Max, Min, MinMax
    from hgq2_amd.regularizers import MonoL1

    w = torch.tensor([-30.0, 0.5, 30.0])
    assert MinMax(-24, 24)(w).tolist() == [-24.0, 0.5, 24.0] and MinMax(-24, 24).bounds() == (-24.0, 24.0)
    assert Min(0)(w).tolist() == [0.0, 0.5, 30.0] and Max(1)(w).tolist() == [-30.0, 0.5, 1.0]
    assert Constant(2)(w).tolist() == [2.0, 2.0, 2.0]
    assert float(MonoL1(1e-2)(w)) == pytest.approx(0.005)


def test_entry_points_validate_arguments_before_any_launch():
    """Bad shapes and null pointers are rejected with the documented codes by host-side checks
    (these calls return before the GPU is touched, so they run anywhere)."""
    from hgq2_amd import _lib

    lib = _lib.load()
    OK, ARG, UNSUPPORTED = 0, -1, -3
    none = ctypes.c_void_p(0)
    # fixed-point quantizer
    assert lib.hgq_quantize_fwd(none, none, none, none, none, none, none, 0, 1, 1, 1, none) == OK   # empty tensor
    assert lib.hgq_quantize_fwd(none, none, none, none, none, none, none, 16, 1, 1, 1, none) == ARG  # null pointers
    assert lib.hgq_quantize_fwd(none, none, none, none, none, none, none, 10, 4, 1, 1, none) == ARG  # 10 % 4 != 0
    assert b'null' in lib.hgq_last_error() or b'multiple' in lib.hgq_last_error()
    # forward + backward in one launch: same checks, and training mode is required
    TRAIN = _lib.MODE_TRAINING | 1
    args9 = [none] * 9
    assert lib.hgq_quantize_fwd_bwd(*args9, 0, 1, 1, TRAIN, none) == OK
    assert lib.hgq_quantize_fwd_bwd(*args9, 16, 16, 1, TRAIN, none) == ARG and b'null' in lib.hgq_last_error()
    one = ctypes.c_void_p(256)  # never dereferenced: the mode check comes before any launch
    assert lib.hgq_quantize_fwd_bwd(*([one] * 9), 16, 16, 1, 1, none) == ARG and b'training' in lib.hgq_last_error()
    assert lib.hgq_quantize_fwd_bwd(*([one] * 9), 10, 4, 1, TRAIN, none) == ARG
    # table softmax: row length, table rows
    assert lib.hgq_qsoftmax_bwd_workspace(1024, 64, 256, 1) > 0
    assert lib.hgq_qsoftmax_bwd_workspace(1024, 300, 1, 0) == -1          # rows longer than 256
    assert lib.hgq_qsoftmax_bwd_workspace(1024, 70, 1, 0) == -1           # > 64 and not a multiple of 4
    assert lib.hgq_qsoftmax_bwd_workspace(1000, 64, 256, 1) == -1         # rows not a multiple of the table rows
    assert lib.hgq_qsoftmax_fwd(none, none, 1024, 300, 1, 1.0, 1e-7, none, none, none, none, none, none, none, none, none) == UNSUPPORTED
    assert lib.hgq_qsoftmax_fwd(none, none, 1024, 64, 1, 1.0, 1e-7, none, none, none, none, none, none, none, none, none) == ARG
    assert lib.hgq_qsoftmax_fwd(none, none, 0, 64, 1, 1.0, 1e-7, none, none, none, none, none, none, none, none, none) == OK
    # convolution geometry
    good = _lib.ConvGeom(4, 8, 8, 3, 3, 3, 1, 1, 0, 0, 1, 1, 6, 6)
    bad = _lib.ConvGeom(4, 8, 8, 3, 3, 3, 0, 1, 0, 0, 1, 1, 6, 6)  # stride 0
    assert lib.hgq_conv2d_bwd_workspace(ctypes.addressof(good), 16) > 0
    assert lib.hgq_conv2d_fwd_workspace(ctypes.addressof(good), 16) == 0
    assert lib.hgq_conv2d_bwd_workspace(ctypes.addressof(bad), 16) == -1
    assert lib.hgq_conv2d_fwd(none, none, none, none, none, ctypes.addressof(bad), 16, 0, none) == ARG
    assert lib.hgq_conv2d_fwd(none, none, none, none, none, ctypes.addressof(good), 16, 7, none) == ARG  # unknown activation
    assert lib.hgq_conv2d_fwd(none, none, none, none, none, ctypes.addressof(good), 16, 0, none) == ARG  # null pointers
    wide = _lib.ConvGeom(8, 1, 1, 4096, 1, 1, 1, 1, 0, 0, 1, 1, 1, 1)
    assert lib.hgq_conv2d_fwd_workspace(ctypes.addressof(wide), 10) > 0   # long contraction, few rows: split along k
    # attention contractions
    assert lib.hgq_attn_scores_fwd(none, none, none, 4, 65, 64, 2, 16, none) == UNSUPPORTED
    assert lib.hgq_attn_scores_fwd(none, none, none, 4, 64, 64, 2, 16, none) == ARG
    assert lib.hgq_attn_combine_bwd(none, none, none, none, none, 0, 64, 64, 2, 16, none) == OK
    # dense
    assert lib.hgq_qdense_bwd(none, none, none, none, 0, none, none, none, none, none, none, 128, 80, 10, 0, 0, none) == UNSUPPORTED
    assert lib.hgq_col_moments_workspace(1000, 64) > 0 and lib.hgq_col_moments_workspace(-1, 64) == -1
    assert lib.hgq_col_moments_fwd(none, 0, 64, none, none, none, none) == ARG
    # contraction + mean over row groups: groups of 32 or 64 rows only, widths multiples of 4 up to 64
    WRAP_TRAIN = _lib.mode_bits('RND', 'WRAP', training=True)
    assert lib.hgq_qdense_fwd_mean_supported(4096, 64, 32, 64, 64, WRAP_TRAIN) == 1
    assert lib.hgq_qdense_fwd_mean_supported(4096, 64, 32, 64, 48, WRAP_TRAIN) == 0    # groups of 48 rows
    assert lib.hgq_qdense_fwd_mean_supported(4096, 64, 30, 0, 64, 0) == 0              # N not a multiple of 4
    assert lib.hgq_qdense_fwd_mean_supported(4100, 64, 32, 0, 64, 0) == 0              # rows not whole groups
    assert lib.hgq_qdense_fwd_mean(none, none, 0, none, none, none, none, none, 4096, 64, 32, 48, 0, 0, none) == UNSUPPORTED
    assert lib.hgq_qdense_fwd_mean(none, none, 0, none, none, none, none, none, 4096, 64, 32, 64, 0, 0, none) == ARG  # null pointers
    assert lib.hgq_qdense_fwd_mean(none, none, 0, none, none, none, none, none, 0, 64, 32, 64, 0, 0, none) == OK
    assert lib.hgq_qdense_bwd_mean_slices(one, none, one, none, 0, one, one, one, 0, 4096, 64, 32, 48, 0, 0, none) == UNSUPPORTED
    assert lib.hgq_qdense_bwd_mean_slices(one, none, one, none, 0, one, one, one, 0, 4096, 64, 32, 0, 0, 0, none) == ARG
    # batch feed, quantizer wrapper, pooling EBOPs, reduction with quantizers attached
    assert lib.hgq_gather_batch(none, 64, none, 8, none, none, none, none, 16, 100, none) == ARG           # null pointers
    assert lib.hgq_gather_batch(one, 6, one, 8, one, one, one, one, 16, 100, none) == ARG and b'32-bit' in lib.hgq_last_error()
    assert lib.hgq_quantizer_scale_div(none, none, 0, 2.0, none) == OK and lib.hgq_quantizer_scale_div(none, none, 8, 2.0, none) == ARG
    assert lib.hgq_quantizer_tail_fwd(one, none, one, 8, 0, 1.0, 1, 0.5, 0, 1.0, 0.0, none) == ARG and b'noise' in lib.hgq_last_error()
    assert lib.hgq_quantizer_tail_bwd(one, one, none, 8, 0, 1.0, 1, 0.5, 0, 1.0, none) == ARG
    assert lib.hgq_sum_ebops(none, 0, 1.0, 1.0, 1.0, none, none, none, none) == UNSUPPORTED
    assert lib.hgq_reduce_slices_quant_multi(none, 1, none, none, none, 0, none) == ARG
    assert lib.hgq_reduce_slices_quant_multi(none, 0, none, none, none, 2, none) == ARG


def test_a_second_thread_inside_a_training_step_is_refused():
    """The launch queues of a step are process-wide (the autograd engine's thread reads them): a second Python thread that
    opens a step while one is open gets an error instead of another step's queue."""
    import threading

    from hgq2_amd import ops

    seen = []

    def other():
        try:
            with ops.side_gradients(None):
                seen.append('entered')
        except RuntimeError as e:
            seen.append(str(e))

    with ops.side_gradients(None):
        t = threading.Thread(target=other)
        t.start()
        t.join()
        with ops.side_gradients(None):  # the same thread may nest
            pass
    assert len(seen) == 1 and 'another thread' in seen[0]
    t = threading.Thread(target=other)  # and once the step is over another thread may run one
    t.start()
    t.join()
    assert seen[1] == 'entered'


def test_beta_controllers_and_ebops_logging():
    """Host-side hooks of reference src/hgq/utils/sugar/{ebops,beta_scheduler,beta_pid}.py on layers built on the CPU
    (no kernel is launched: the hooks only read `_ebops` and assign `_beta`)."""
    from math import log10

    from hgq2_amd.core import Sequential
    from hgq2_amd.layers import QDense
    from hgq2_amd.utils.sugar import PID, BetaPID, BetaScheduler, FreeEBOPs, PieceWiseSchedule, fit

    sched = PieceWiseSchedule([(10, 1e-5, 'log'), (0, 0.0, 'linear'), (20, 1e-3, 'constant')])
    assert sched(0) == 0.0 and abs(sched(5) - 5e-6) < 1e-12 and abs(sched(10) - 1e-5) < 1e-12
    assert abs(sched(15) - 1e-4) < 1e-9 and sched(20) == 1e-3 and sched(300) == 1e-3
    pid = PID(2.0, 0.5, 0.25, neg=False)
    assert pid(1.0, 0.0) == 2.0 + 0.5 + 0.25 and pid(1.0, 0.5) == 1.0 + 0.75 - 0.125
    layers = [QDense(8), QDense(4)]
    model = Sequential(layers)
    shape = (None, 16)
    for layer in layers:
        layer.build(shape)
        shape = (None, layer.units)
    counters = iter([(1000, 3000), (800, 2400), (500, 1000), (100, 300)])

    def step(_):
        a, b = next(counters)
        with torch.no_grad():
            layers[0]._ebops.view(torch.int32).fill_(a), layers[1]._ebops.view(torch.int32).fill_(b)
        return 1.5

    history = fit(model, step, lambda epoch: [0], 4, [BetaScheduler(sched), FreeEBOPs()])
    assert [h['ebops'] for h in history] == [4000, 3200, 1500, 400]
    assert [h['beta'] for h in history] == [sched(e) for e in range(4)] and history[0]['loss'] == 1.5
    assert float(layers[1]._beta) == pytest.approx(sched(3))
    # the PID controller: idle during warm-up, then its first output repeats the beta in force (integral initialisation),
    # and a model above its EBOPs target gets a larger beta the next epoch
    counters = iter([(1000, 3000)] * 6)
    ctl = BetaPID(target_ebops=2000.0, init_beta=1e-6, p=1.0, i=0.1, warmup=2, log=True)
    history = fit(model, step, lambda epoch: [0], 5, [ctl])
    assert float(layers[0]._beta) == pytest.approx(history[-1]['beta'])
    assert history[0]['beta'] == pytest.approx(1e-6) and history[2]['beta'] == pytest.approx(1e-6, rel=1e-6)
    err = log10(4000 / 2000)
    assert history[3]['beta'] == pytest.approx(10 ** (log10(1e-6) + 0.1 * err), rel=1e-6) and history[4]['beta'] > history[3]['beta']
    assert all(h['ebops'] == 4000 for h in history)


def test_reciprocal_index_arithmetic_is_exact_on_the_ranges_the_kernels_use():
    """The staging maps of the fused dense kernels divide by a 16-bit reciprocal (ids below 1024, divisors up to 16);
    the staging loops of the small-channel convolution and the EBOPs kernels by a float reciprocal (values below
    2**21).  Both claim to equal integer division on those ranges."""
    import numpy as np

    for w4 in range(1, 17):
        rcp = (65536 + w4 - 1) // w4
        ids = np.arange(1024, dtype=np.uint64)
        assert np.array_equal((ids * rcp) >> 16, ids // w4), w4
    c = np.arange(1 << 21, dtype=np.uint32)
    for d in (1, 2, 3, 5, 7, 12, 31, 32, 33, 68, 272, 340, 1088, 3872, 30719):
        inv = np.float32(1.0) / np.float32(d)
        q = ((c.astype(np.float32) + np.float32(0.5)) * inv).astype(np.uint32)
        assert np.array_equal(q, c // d), d


def test_matrix_instruction_choice_from_the_environment():
    """`HGQ_MATRIX_INSTRUCTION=fp32` starts the package with the contractions on the fp32 matrix instruction; without it the
    bf16-part kernels are the default (`hgq_dense_use_bf16_parts`: a negative argument only reads the setting)."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = 'from hgq2_amd import _lib; print(_lib.load().hgq_dense_use_bf16_parts(-1))'
    for value, want in ((None, '1'), ('fp32', '0'), ('bf16', '1')):
        env = {k: v for k, v in os.environ.items() if k != 'HGQ_MATRIX_INSTRUCTION'}
        if value is not None:
            env['HGQ_MATRIX_INSTRUCTION'] = value
        out = subprocess.run([sys.executable, '-c', code], cwd=root, env=env, capture_output=True, text=True, timeout=120)
        assert out.returncode == 0, out.stderr
        assert out.stdout.strip().splitlines()[-1] == want, (value, out.stdout)


def test_fit_checks_its_arguments_and_seed_generators_count_on_the_host():
    """Host logic only: `train.fit` refuses CPU tensors (the product has no CPU path) and mismatched sample counts before
    anything is built; a seed generator used without a device keeps the host counter 1, 2, 3, ... and never creates the
    device-side one."""
    from hgq2_amd.quantizer.fixed_point_ops import SeedGenerator
    from hgq2_amd.train import fit

    x, y = torch.zeros(8, 4), torch.zeros(8, dtype=torch.int64)
    with pytest.raises(ValueError, match='GPU'):
        fit(object(), x, y)
    with pytest.raises(ValueError, match='same'):
        fit(object(), x, y[:5])
    gen = SeedGenerator(9)
    assert [gen.next() for _ in range(3)] == [(9, 1), (9, 2), (9, 3)]
    assert gen._base is None and gen.offset == 3
    assert gen.next(torch.device('cpu')) == (9, 4)
