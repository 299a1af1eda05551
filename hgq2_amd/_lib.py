"""ctypes binding of ``libhgq_hip.so`` (declared in ``include/hgq_hip.h``).

There is no CPU fallback: if the library is missing or a call fails, this raises.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, 'libhgq_hip.so')

# mode bits, mirrored from include/hgq_hip.h
TRN, RND, RND_CONV = 0, 1, 2
S_RND, S_RND_CONV = 3, 4  # stochastic in training (hgq_quantize_*_stochastic), RND / RND_CONV otherwise
WRAP, SAT, SAT_SYM = 0, 1, 2
MODE_TRAINING = 1 << 8
MODE_KBI = 1 << 9
MODE_ROUND_PARAMS = 1 << 10
MODE_K_U8 = 1 << 11
MODE_SYMMETRIC = 1 << 12
MODE_TRACING = 1 << 13
MODE_TRACK_INPUT = 1 << 14
ACT_NONE, ACT_RELU = 0, 1

ROUND_MODES = {'TRN': TRN, 'RND': RND, 'RND_CONV': RND_CONV}
OVERFLOW_MODES = {'WRAP': WRAP, 'SAT': SAT, 'SAT_SYM': SAT_SYM}

ERRORS = {-1: 'HGQ_ERR_ARG', -2: 'HGQ_ERR_LAUNCH', -3: 'HGQ_ERR_UNSUPPORTED'}
ERR_ARG, ERR_LAUNCH, ERR_UNSUPPORTED = -1, -2, -3
STATIC_SCRATCH_FLOATS = 1 << 18  # HGQ_STATIC_SCRATCH_FLOATS of include/hgq_hip.h

# name -> (restype, argtypes); exactly the declarations of include/hgq_hip.h
SIGNATURES = {
    'hgq_version': (c_int, []),
    'hgq_last_error': (c_char_p, []),
    'hgq_quantize_fwd': (c_int, [c_void_p] * 7 + [c_int64, c_int64, c_int64, c_int, c_void_p]),
    'hgq_quantize_tracker_slices': (c_int64, [c_int64, c_int64, c_int64]),
    'hgq_quantize_fwd_sliced': (c_int, [c_void_p] * 7 + [c_int64, c_int64, c_int64, c_int64, c_int, c_void_p]),
    'hgq_quantize_bwd': (c_int, [c_void_p] * 8 + [c_int64, c_int64, c_int64, c_int, c_void_p]),
    'hgq_quantize_fwd_stochastic': (c_int, [c_void_p] * 7 + [c_int64, c_int64, c_int64, c_int, ctypes.c_uint64, ctypes.c_uint64, c_void_p]),
    'hgq_quantize_bwd_stochastic': (c_int, [c_void_p] * 8 + [c_int64, c_int64, c_int64, c_int, ctypes.c_uint64, ctypes.c_uint64, c_void_p]),
    'hgq_quantize_fwd_stochastic_at': (c_int, [c_void_p] * 7 + [c_int64, c_int64, c_int64, c_int, ctypes.c_uint64, ctypes.c_uint64, c_void_p, c_void_p,
                                               c_void_p]),
    'hgq_quantize_bwd_stochastic_at': (c_int, [c_void_p] * 8 + [c_int64, c_int64, c_int64, c_int, ctypes.c_uint64, c_void_p, c_void_p]),
    'hgq_counters_advance': (c_int, [c_void_p, c_void_p, c_int, c_void_p]),
    'hgq_wrap_track_i': (c_int, [c_void_p] * 2 + [c_int] + [c_void_p] * 3 + [c_int64, c_float, c_float, c_float, c_int, c_void_p]),
    'hgq_qdense_fwd_parts': (c_int, [c_int64]),
    'hgq_qdense_bwd_workspace': (c_int64, [c_int64, c_int, c_int, c_int64]),
    'hgq_qdense_fwd': (c_int, [c_void_p] * 4 + [c_int64] + [c_void_p] * 4 + [c_int64, c_int, c_int, c_int, c_int, c_void_p]),
    'hgq_qdense_fwd_oq_supported': (c_int, [c_int64, c_int, c_int, c_int64, c_int64, c_int, c_int]),
    'hgq_qdense_fwd_oq': (c_int, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64] + [c_void_p] * 4
                          + [c_int64, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    'hgq_qdense_bwd': (c_int, [c_void_p] * 4 + [c_int64] + [c_void_p] * 6 + [c_int64, c_int, c_int, c_int, c_int, c_void_p]),
    'hgq_qdense_fwd_mean_supported': (c_int, [c_int64, c_int, c_int, c_int64, c_int64, c_int]),
    'hgq_qdense_fwd_mean': (c_int, [c_void_p, c_void_p, c_int64] + [c_void_p] * 5 + [c_int64, c_int, c_int, c_int64, c_int, c_int, c_void_p]),
    'hgq_qdense_bwd_mean': (c_int, [c_void_p] * 4 + [c_int64] + [c_void_p] * 6 + [c_int64, c_int, c_int, c_int64, c_int, c_int, c_void_p]),
    'hgq_qdense_bwd_mean_slices': (c_int, [c_void_p] * 4 + [c_int64] + [c_void_p] * 3 + [c_int, c_int64, c_int, c_int, c_int64, c_int, c_int,
                                           c_void_p]),
    'hgq_dense_ebops': (
        c_int,
        [c_void_p, c_int, c_float, c_void_p, c_void_p] + [c_void_p] * 3 + [c_int64, c_int, c_int] + [c_void_p] * 4
        + [c_float, c_float, c_float, c_float, c_int, c_int, c_int] + [c_void_p] * 5 + [c_void_p],
    ),
    'hgq_ebops_finish_fwd': (c_int, [c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_void_p]),
    'hgq_ebops_finish_bwd': (c_int, [c_void_p, c_void_p, c_float, c_void_p, c_void_p]),
    'hgq_lut_ebops': (c_int, [c_void_p, c_void_p, c_int64, c_float, c_float, c_void_p, c_void_p, c_void_p, c_void_p]),
    'hgq_sum_ebops': (c_int, [c_void_p, c_int64, c_float, c_float, c_float, c_void_p, c_void_p, c_void_p, c_void_p]),
    'hgq_softmax_ebops': (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_float, c_float, c_void_p, c_void_p, c_void_p, c_void_p]),
    'hgq_mha_ebops': (c_int, [c_void_p] * 4 + [c_int] * 5 + [c_float, c_float, c_void_p, c_void_p, c_void_p, c_void_p]),
    'hgq_qbits_fwd': (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p]),
    'hgq_qbits_bwd': (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_void_p, c_void_p, c_void_p]),
    'hgq_bn_fold_fwd': (c_int, [c_void_p] * 5 + [c_int, c_float] + [c_void_p] * 4 + [c_float, c_float, c_int, c_int, c_void_p]),
    'hgq_bn_fold_quant_fwd': (c_int, [c_void_p] * 5 + [c_int, c_float] + [c_void_p] * 6 + [c_float, c_float, c_int, c_int, c_void_p]),
    'hgq_bn_fold_quant_bwd': (c_int, [c_void_p] * 5 + [c_int, c_float] + [c_void_p] * 13 + [c_int, c_int, c_void_p]),
    'hgq_bn_fold_bwd': (c_int, [c_void_p] * 4 + [c_int, c_float] + [c_void_p] * 7 + [c_int, c_int, c_void_p]),
    'hgq_qdense_moments_workspace': (c_int64, [c_int64, c_int, c_int, c_int64]),
    'hgq_qdense_moments_fwd': (c_int, [c_void_p, c_void_p, c_int64, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p]),
    'hgq_qdense_moments_bwd': (c_int, [c_void_p, c_void_p, c_int64, c_int] + [c_void_p] * 8 + [c_int64, c_int, c_int, c_void_p]),
    'hgq_dense_moments_workspace': (c_int64, [c_int64, c_int, c_int]),
    'hgq_dense_moments_fwd': (c_int, [c_void_p] * 5 + [c_int64, c_int, c_int, c_void_p]),
    'hgq_dense_moments_bwd': (c_int, [c_void_p] * 7 + [c_int64, c_int, c_int, c_void_p]),
    'hgq_mse_workspace': (c_int64, []),
    'hgq_mse_fwd': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    'hgq_mse_bwd': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    'hgq_mse_fwd_bwd': (c_int, [c_void_p] * 5 + [c_int64, c_void_p]),
    'hgq_sparse_ce_fwd_bwd': (c_int, [c_void_p] * 4 + [c_int64, c_int, c_void_p, c_void_p]),
    'hgq_gather_batch': (c_int, [c_void_p, c_int64, c_void_p, c_int64] + [c_void_p] * 4 + [c_int64, c_int64, c_void_p]),
    'hgq_sgd_update': (c_int, [c_void_p, c_void_p, c_int64, c_float, c_float, c_float, c_float, c_void_p]),
    'hgq_sgd_update_multi': (c_int, [c_void_p, c_int, c_float, c_void_p]),
    'hgq_sgd_update_multi_sum': (c_int, [c_void_p, c_int, c_float, c_void_p, c_int, c_void_p, c_void_p]),
    'hgq_quantize_bwd_workspace': (c_int64, [c_int64, c_int64, c_int64]),
    'hgq_quantize_bwd_sliced': (c_int, [c_void_p] * 9 + [c_int64, c_int64, c_int64, c_int, c_void_p]),
    'hgq_quantize_bwd_slice_count': (c_int64, [c_int64, c_int64, c_int64]),
    'hgq_dense_use_bf16_parts': (c_int, [c_int]),
    'hgq_quantize_bwd_slices': (c_int, [c_void_p] * 6 + [c_int, c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p]),
    'hgq_conv2d_ebops_q': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_float, c_float, c_float, c_void_p, c_void_p, c_void_p, c_void_p]),
    'hgq_dense_ebops_multi': (c_int, [c_void_p, c_int, c_void_p]),
    'hgq_wrap_track_i_multi': (c_int, [c_void_p, c_int, c_void_p]),
    'hgq_qdense_bwd_slices': (c_int, [c_void_p] * 4 + [c_int64] + [c_void_p] * 3 + [c_int, c_int64, c_int, c_int, c_int, c_int, c_void_p]),
    'hgq_reduce_slices_multi': (c_int, [c_void_p, c_int, c_void_p]),
    'hgq_reduce_slices_quant_multi': (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p]),
    'hgq_stream_probe': (c_int, [c_void_p] * 7 + [c_int, c_int, c_int64, c_void_p]),
    'hgq_quantize_bwd_static': (c_int, [c_void_p] * 8 + [c_int64, c_int64, c_int64, c_int, c_void_p]),
    'hgq_quantize_fwd_bwd': (c_int, [c_void_p] * 9 + [c_int64, c_int64, c_int64, c_int, c_void_p]),
    'hgq_quantize_fwd_multi': (c_int, [c_void_p, c_int, c_void_p]),
    'hgq_quantize_bwd_multi': (c_int, [c_void_p, c_int, c_void_p]),
    'hgq_gdense_supported': (c_int, [c_int64, c_int, c_int, c_int]),
    'hgq_gdense_fwd': (c_int, [c_void_p] * 4 + [c_int64, c_int, c_int, c_int, c_int, c_void_p]),
    'hgq_gdense_bwd_workspace': (c_int64, [c_int64, c_int, c_int, c_int, c_int]),
    'hgq_gdense_bwd': (c_int, [c_void_p] * 8 + [c_int64, c_int, c_int, c_int, c_int, c_void_p]),
    'hgq_affine_rows_fwd': (c_int, [c_void_p] * 4 + [c_int64, c_int, c_void_p]),
    'hgq_affine_rows_bwd_workspace': (c_int64, [c_int64, c_int]),
    'hgq_affine_rows_bwd': (c_int, [c_void_p] * 7 + [c_int64, c_int, c_void_p]),
    'hgq_quantizer_scale_div': (c_int, [c_void_p, c_void_p, c_int64, c_float, c_void_p]),
    'hgq_quantizer_tail_fwd': (c_int, [c_void_p] * 3 + [c_int64, c_int, c_float, c_int, c_float, c_int, c_float, c_float, c_void_p]),
    'hgq_quantizer_tail_bwd': (c_int, [c_void_p] * 3 + [c_int64, c_int, c_float, c_int, c_float, c_int, c_float, c_void_p]),
    'hgq_mean_mid_fwd': (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p]),
    'hgq_mean_mid_bwd': (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p]),
    'hgq_sum_scalars': (c_int, [c_void_p, c_int, c_void_p, c_void_p]),
    'hgq_mlp_workspace': (c_int64, [c_void_p, c_int, c_int64]),
    'hgq_mlp_train_step': (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int64, c_float, c_void_p, c_void_p, c_void_p]),
    'hgq_mlp_train_step_cached': (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int64, c_float, c_void_p, c_void_p, c_int, c_void_p]),
    'hgq_fill_u32': (c_int, [c_void_p, ctypes.c_uint32, c_int64, c_void_p]),
    'hgq_qsoftmax_fwd': (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int64, c_float, c_float] + [c_void_p] * 5
                         + [c_void_p] * 3 + [c_void_p]),
    'hgq_qsoftmax_bwd_workspace': (c_int64, [c_int64, c_int, c_int64, c_int]),
    'hgq_qsoftmax_bwd': (c_int, [c_void_p] * 3 + [c_int64, c_int, c_int64, c_float, c_float] + [c_void_p] * 5
                         + [c_void_p] * 4 + [c_void_p]),
    'hgq_qattention_fwd': (c_int, [c_void_p] * 4 + [c_int] * 5 + [c_int64, c_float, c_float] + [c_void_p] * 5 + [c_void_p] * 3
                           + [c_void_p, c_void_p, c_int, c_int, c_void_p]),
    'hgq_qattention_fwd_workspace': (c_int64, [c_int] * 5 + [c_int64, c_int]),
    'hgq_qattention_bwd_workspace': (c_int64, [c_int] * 5 + [c_int64, c_int]),
    'hgq_qattention_bwd': (c_int, [c_void_p] * 7 + [c_int] * 5 + [c_int64, c_float, c_float] + [c_void_p] * 5 + [c_void_p] * 4
                           + [c_void_p, c_int, c_int, c_void_p]),
    'hgq_attn_scores_fwd': (c_int, [c_void_p] * 3 + [c_int] * 5 + [c_void_p]),
    'hgq_attn_scores_bwd': (c_int, [c_void_p] * 5 + [c_int] * 5 + [c_void_p]),
    'hgq_attn_combine_fwd': (c_int, [c_void_p] * 3 + [c_int] * 5 + [c_void_p]),
    'hgq_attn_combine_bwd': (c_int, [c_void_p] * 5 + [c_int] * 5 + [c_void_p]),
    'hgq_pool2d_fwd': (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_void_p]),
    'hgq_pool2d_bwd': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p]),
    'hgq_col_moments_workspace': (c_int64, [c_int64, c_int]),
    'hgq_col_moments_fwd': (c_int, [c_void_p, c_int64, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    'hgq_col_moments_bwd': (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_void_p, c_void_p]),
    'hgq_conv2d_ebops': (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    'hgq_conv2d_fwd_workspace': (c_int64, [c_void_p, c_int]),
    'hgq_conv2d_fwd': (c_int, [c_void_p] * 6 + [c_int, c_int, c_void_p]),
    'hgq_conv2d_bwd_workspace': (c_int64, [c_void_p, c_int]),
    'hgq_conv2d_bwd': (c_int, [c_void_p] * 9 + [c_int, c_int, c_void_p]),
    'hgq_conv2d_bwd_slice_count': (c_int64, [c_void_p, c_int]),
    'hgq_conv2d_bwd_slices': (c_int, [c_void_p] * 7 + [c_int, c_int, c_void_p]),
    'hgq_conv2d_maxpool_bwd_supported': (c_int, [c_void_p, c_int]),
    'hgq_conv2d_maxpool_fwd': (c_int, [c_void_p] * 6 + [c_int, c_int, c_void_p]),
    'hgq_conv2d_maxpool_bwd': (c_int, [c_void_p] * 9 + [c_int, c_int, c_int, c_void_p]),
    'hgq_conv2d_maxpool_fwd_coded': (c_int, [c_void_p] * 6 + [c_int, c_int, c_void_p]),
    'hgq_conv2d_maxpool_bwd_coded': (c_int, [c_void_p] * 9 + [c_int, c_int, c_int, c_void_p]),
}


class ConvGeom(ctypes.Structure):
    """``hgq_conv_geom`` of include/hgq_hip.h."""

    _fields_ = [(n, c_int) for n in ('B', 'H', 'W', 'C', 'kh', 'kw', 'sy', 'sx', 'py', 'px', 'dly', 'dlx', 'OH', 'OW')]


class QDesc(ctypes.Structure):
    """``hgq_qdesc`` of include/hgq_hip.h: one quantizer's raw variables and mode bits."""

    _fields_ = [('k', c_void_p), ('i', c_void_p), ('fb', c_void_p), ('mode', c_int)]



class BitsDesc(ctypes.Structure):
    """``hgq_bits_desc`` of include/hgq_hip.h: a quantizer's bit-width view and where its gradients go."""

    _fields_ = [('k', c_void_p), ('i', c_void_p), ('fb', c_void_p), ('size', c_int64), ('inner', c_int64), ('kbi', c_int),
                ('add_mode', c_int), ('g_i', c_void_p), ('g_fb', c_void_p)]


class MlpLayer(ctypes.Structure):
    """``hgq_mlp_layer`` of include/hgq_hip.h."""

    _fields_ = (
        [(n, c_int) for n in ('K', 'N', 'act', 'mode_in', 'mode_ker', 'mode_bias')]
        + [(n, c_void_p) for n in ('w', 'bias', 'k_in', 'i_in', 'f_in', 'k_ker', 'b_ker', 'i_ker', 'k_bias', 'b_bias', 'i_bias')]
        + [('decay', c_float), ('beta', c_void_p), ('ebops', c_void_p), ('par_factor', c_float), ('n_parallel', c_float), ('ebops_factor', c_float), ('bias_size', c_float)]
        + [(n, c_float) for n in ('f_in_l1', 'f_in_lo', 'f_in_hi', 'b_ker_l1', 'b_ker_lo', 'b_ker_hi', 'i_ker_l1', 'i_ker_lo',
                                  'i_ker_hi', 'b_bias_l1', 'b_bias_lo', 'b_bias_hi', 'i_bias_l1', 'i_bias_lo', 'i_bias_hi')]
        + [('train_i_ker', c_int), ('train_i_bias', c_int)]
    )


_lib = None


class HGQLibraryError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Load the HIP library; raise if it has not been built (``python -c 'import __graft_entry__ as g; g.build()'``)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise HGQLibraryError(
            f'{LIB_PATH} not found: the HIP extension is not built. Run `make -C hgq2_amd/csrc` '
            '(or __graft_entry__.build()). There is no CPU fallback.'
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    if os.environ.get('HGQ_MATRIX_INSTRUCTION', '').lower() == 'fp32':
        lib.hgq_dense_use_bf16_parts(0)  # contractions on the fp32 matrix instruction instead of bf16 parts
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().hgq_last_error()
        raise HGQLibraryError(f'{what} failed with {ERRORS.get(rc, rc)}: {msg.decode() if msg else ""}')


def mode_bits(round_mode: str, overflow_mode: str, *, training=False, kbi=False, round_params=False, k_u8=False,
              symmetric=False, tracing=False, track_input=False) -> int:
    rm = round_mode.upper()
    if rm.startswith('S_'):
        rm = rm[2:]
    try:
        m = ROUND_MODES[rm] | (OVERFLOW_MODES[overflow_mode.upper()] << 4)
    except KeyError as e:
        raise ValueError(f'unsupported round/overflow mode {round_mode}/{overflow_mode}') from e
    if training:
        m |= MODE_TRAINING
    if kbi:
        m |= MODE_KBI
    if round_params:
        m |= MODE_ROUND_PARAMS
    if k_u8:
        m |= MODE_K_U8
    if symmetric:
        m |= MODE_SYMMETRIC
    if tracing:
        m |= MODE_TRACING
    if track_input:
        m |= MODE_TRACK_INPUT
    return m
