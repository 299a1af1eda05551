"""``torch.library`` operators over the C ABI of ``libhgq_hip.so`` and their autograd wrappers.

Layering: ``hgq::*`` custom operators are thin, validated launches of one C-ABI entry point
(outputs allocated with torch, kernels enqueued on torch's current stream); the
``torch.autograd.Function`` classes below pair each forward operator with its backward
operator.  There is no CPU implementation: tensors must live on a GPU and a missing library
raises.
"""

from __future__ import annotations

import ctypes
import threading
from typing import Sequence

import torch
from torch import Tensor

from . import _lib

__all__ = ['quantize', 'wrap_track_i_', 'qdense', 'dense_ebops', 'sparse_ce', 'sgd_update_', 'sgd_update_multi_', 'qsoftmax', 'conv2d', 'matmul_bias_act', 'col_moments', 'attn_scores', 'attn_combine', 'ATTN_MAX', 'pool2d', 'conv2d_ebops', 'conv_geometry', 'conv2d_ebops_supported', 'mse', 'dense_moments', 'dense_moments_supported', 'bn_fold', 'qbits', 'ebops_finish', 'qattention', 'qattention_supported', 'bits_ebops', 'gdense', 'gdense_supported', 'affine_rows']


def _ptr(t: Tensor | None):
    return ctypes.c_void_p(t.data_ptr()) if t is not None and t.numel() > 0 else ctypes.c_void_p(0)


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need(cond: bool, msg: str):
    if not cond:
        raise ValueError(msg)


_F32 = torch.float32


# The queues and flags further down (deferred launches, the second stream's branch, the gradient sink) belong to the
# ONE training step that is running: they are process-wide on purpose, because the backward functions that read them run
# on the autograd engine's device thread, not on the thread that opened them.  Two Python threads driving model calls at
# the same time would mix their queues, so the second one is refused loudly.
_STEP_OWNER = {'thread': None, 'depth': 0}


def _claim_step(what: str):
    me = threading.get_ident()
    if _STEP_OWNER['depth'] and _STEP_OWNER['thread'] != me:
        raise RuntimeError(f'{what}: another thread is inside a model call or training step of this package; its launch queues '
                           'are process-wide (the autograd engine reads them from its own thread), so steps must not overlap')
    _STEP_OWNER['thread'] = me
    _STEP_OWNER['depth'] += 1


def _release_step():
    _STEP_OWNER['depth'] -= 1
    if _STEP_OWNER['depth'] <= 0:
        _STEP_OWNER['depth'], _STEP_OWNER['thread'] = 0, None


def _check_f32(name: str, t: Tensor):
    # (the messages are built only on failure: these checks run a hundred times per training step)
    if t.is_cuda and t.dtype is _F32 and t.is_contiguous():
        return
    _need(t.is_cuda, f'{name} must be a GPU tensor (there is no CPU implementation), got device {t.device}')
    _need(t.dtype == torch.float32, f'{name} must be float32, got {t.dtype}')
    _need(t.is_contiguous(), f'{name} must be contiguous')


def _check_k(name: str, t: Tensor):
    if t.is_cuda and (t.dtype is _F32 or t.dtype is torch.uint8) and t.is_contiguous():
        return
    _need(t.is_cuda, f'{name} must be a GPU tensor')
    _need(t.dtype in (torch.float32, torch.uint8), f'{name} must be float32 or uint8, got {t.dtype}')
    _need(t.is_contiguous(), f'{name} must be contiguous')


def _kmode(mode: int, k: Tensor) -> int:
    return (mode | _lib.MODE_K_U8) if k.dtype == torch.uint8 else (mode & ~_lib.MODE_K_U8)


# ======================================================================================
# raw operators (one C-ABI call each)
# ======================================================================================
@torch.library.custom_op('hgq::quantize_fwd', mutates_args=())
def quantize_fwd(x: Tensor, k: Tensor, i: Tensor, fb: Tensor, mode: int, bw_inner: int, track: bool) -> tuple[Tensor, Tensor, Tensor]:
    _check_f32('x', x), _check_k('k', k), _check_f32('i', i), _check_f32('fb', fb)
    bw_size = i.numel()
    _need(k.numel() == bw_size and fb.numel() == bw_size, 'k, i, f must have the same number of elements')
    n = x.numel()
    _need(bw_size >= 1 and bw_inner >= 1 and (n == 0 or n % (bw_size * bw_inner) == 0),
          f'x has {n} elements, not a multiple of bw_size*bw_inner = {bw_size}*{bw_inner}')
    y = torch.empty_like(x)
    lib = _lib.load()
    slices = lib.hgq_quantize_tracker_slices(n, bw_size, bw_inner) if track and n else 0
    if slices and all(t.data_ptr() % 16 == 0 for t in (x, y, k, i, fb)):
        # trackers as one slice per row chunk ([slices, bw_size]): no clearing launch, no atomics
        amax = torch.empty(slices * bw_size, dtype=torch.int32, device=x.device)
        neg = torch.empty(slices * bw_size, dtype=torch.int32, device=x.device)
        rc = lib.hgq_quantize_fwd_sliced(_ptr(x), _ptr(k), _ptr(i), _ptr(fb), _ptr(y), _ptr(amax), _ptr(neg), slices, n, bw_size,
                                         bw_inner, _kmode(mode, k), _stream())
        _lib.check(rc, 'hgq_quantize_fwd_sliced')
        return y, amax, neg
    amax = torch.empty(bw_size if track else 0, dtype=torch.int32, device=x.device)
    neg = torch.empty(bw_size if track else 0, dtype=torch.int32, device=x.device)
    rc = lib.hgq_quantize_fwd(_ptr(x), _ptr(k), _ptr(i), _ptr(fb), _ptr(y), _ptr(amax), _ptr(neg), n, bw_size,
                              bw_inner, _kmode(mode, k), _stream())
    _lib.check(rc, 'hgq_quantize_fwd')
    return y, amax, neg


@quantize_fwd.register_fake
def _(x, k, i, fb, mode, bw_inner, track):
    m = i.numel() if track else 0
    if m and x.numel():
        m *= max(int(_lib.load().hgq_quantize_tracker_slices(x.numel(), i.numel(), bw_inner)), 1)
    return torch.empty_like(x), x.new_empty(m, dtype=torch.int32), x.new_empty(m, dtype=torch.int32)


@torch.library.custom_op('hgq::quantize_bwd', mutates_args=())
def quantize_bwd(dy: Tensor, x: Tensor, k: Tensor, i: Tensor, fb: Tensor, mode: int, bw_inner: int, need_dx: bool,
                 need_di: bool) -> tuple[Tensor, Tensor, Tensor]:
    _check_f32('dy', dy), _check_f32('x', x), _check_k('k', k), _check_f32('i', i), _check_f32('fb', fb)
    _need(dy.numel() == x.numel(), 'dy and x differ in size')
    dx = torch.empty_like(x) if need_dx else x.new_empty(0)
    di = torch.empty_like(i) if need_di else i.new_empty(0)
    dfb = torch.empty_like(fb)
    lib = _lib.load()
    n_ws = lib.hgq_quantize_bwd_workspace(x.numel(), i.numel(), bw_inner)
    if n_ws and all(t.data_ptr() % 16 == 0 for t in (dy, x, k, i, fb, dx)):
        # bit-width gradients as one slice per row chunk, added in a fixed order: no clearing launch, no atomics
        ws = torch.empty(n_ws, dtype=torch.float32, device=x.device)
        rc = lib.hgq_quantize_bwd_sliced(_ptr(dy), _ptr(x), _ptr(k), _ptr(i), _ptr(fb), _ptr(dx), _ptr(di), _ptr(dfb), _ptr(ws),
                                         x.numel(), i.numel(), bw_inner, _kmode(mode, k), _stream())
        _lib.check(rc, 'hgq_quantize_bwd_sliced')
        return dx, di, dfb
    rc = lib.hgq_quantize_bwd(_ptr(dy), _ptr(x), _ptr(k), _ptr(i), _ptr(fb), _ptr(dx), _ptr(di), _ptr(dfb),
                              x.numel(), i.numel(), bw_inner, _kmode(mode, k), _stream())
    _lib.check(rc, 'hgq_quantize_bwd')
    return dx, di, dfb


@torch.library.custom_op('hgq::quantize_fwd_bwd', mutates_args=())
def quantize_fwd_bwd(x: Tensor, k: Tensor, i: Tensor, fb: Tensor, dy: Tensor, mode: int, bw_inner: int) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    """Training-mode forward and surrogate backward in one launch: ``(y, dx, di, dfb)`` for a caller that holds the upstream
    gradient ``dy`` when it quantizes.  ``mode`` must carry MODE_TRAINING."""
    _check_f32('x', x), _check_k('k', k), _check_f32('i', i), _check_f32('fb', fb), _check_f32('dy', dy)
    bw_size = i.numel()
    _need(k.numel() == bw_size and fb.numel() == bw_size, 'k, i, f must have the same number of elements')
    _need(dy.numel() == x.numel(), 'dy and x differ in size')
    n = x.numel()
    _need(bw_size >= 1 and bw_inner >= 1 and (n == 0 or n % (bw_size * bw_inner) == 0),
          f'x has {n} elements, not a multiple of bw_size*bw_inner = {bw_size}*{bw_inner}')
    y, dx, di, dfb = torch.empty_like(x), torch.empty_like(x), torch.empty_like(i), torch.empty_like(fb)
    rc = _lib.load().hgq_quantize_fwd_bwd(_ptr(x), _ptr(k), _ptr(i), _ptr(fb), _ptr(dy), _ptr(y), _ptr(dx), _ptr(di), _ptr(dfb), n,
                                          bw_size, bw_inner, _kmode(mode, k), _stream())
    _lib.check(rc, 'hgq_quantize_fwd_bwd')
    return y, dx, di, dfb


@quantize_fwd_bwd.register_fake
def _(x, k, i, fb, dy, mode, bw_inner):
    return torch.empty_like(x), torch.empty_like(x), torch.empty_like(i), torch.empty_like(fb)


@torch.library.custom_op('hgq::quantize_bwd_slices', mutates_args=())
def quantize_bwd_slices(dy: Tensor, x: Tensor, k: Tensor, i: Tensor, fb: Tensor, mode: int, bw_inner: int, need_dx: bool,
                        need_di: bool) -> tuple[Tensor, Tensor]:
    """The data gradient and the slices ``[n_slices, bw (fb) + bw (i, with need_di)]`` of the bit-width gradients, left for
    a joint reduction; only for shapes ``quantize_bwd_slices_supported`` accepts."""
    _check_f32('dy', dy), _check_f32('x', x), _check_k('k', k), _check_f32('i', i), _check_f32('fb', fb)
    _need(dy.numel() == x.numel(), 'dy and x differ in size')
    lib = _lib.load()
    n_sl = lib.hgq_quantize_bwd_slice_count(x.numel(), i.numel(), bw_inner)
    _need(n_sl > 0, 'shape outside the sliced backward')
    dx = torch.empty_like(x) if need_dx else x.new_empty(0)
    ws = torch.empty((n_sl, i.numel() * (2 if need_di else 1)), dtype=torch.float32, device=x.device)
    rc = lib.hgq_quantize_bwd_slices(_ptr(dy), _ptr(x), _ptr(k), _ptr(i), _ptr(fb), _ptr(dx), int(need_di), _ptr(ws), x.numel(), i.numel(),
                                     bw_inner, _kmode(mode, k), _stream())
    _lib.check(rc, 'hgq_quantize_bwd_slices')
    return dx, ws


@quantize_bwd_slices.register_fake
def _(dy, x, k, i, fb, mode, bw_inner, need_dx, need_di):
    n_sl = max(int(_lib.load().hgq_quantize_bwd_slice_count(x.numel(), i.numel(), bw_inner)), 1)
    return (torch.empty_like(x) if need_dx else x.new_empty(0), x.new_empty((n_sl, i.numel() * (2 if need_di else 1))))


def quantize_bwd_slices_supported(dy: Tensor, x: Tensor, k: Tensor, i: Tensor, fb: Tensor, bw_inner: int) -> bool:
    return (x.numel() > 0 and all(t.data_ptr() % 16 == 0 for t in (dy, x, k, i, fb))
            and _lib.load().hgq_quantize_bwd_slice_count(x.numel(), i.numel(), bw_inner) > 0)


@quantize_bwd.register_fake
def _(dy, x, k, i, fb, mode, bw_inner, need_dx, need_di):
    return (torch.empty_like(x) if need_dx else x.new_empty(0), torch.empty_like(i) if need_di else i.new_empty(0),
            torch.empty_like(fb))


@torch.library.custom_op('hgq::wrap_track_i', mutates_args=('i_var', 'k_var'))
def wrap_track_i_op(amax: Tensor, anyneg: Tensor, n_parts: int, i_var: Tensor, fb: Tensor, k_var: Tensor, decay: float,
                    c_lo: float, c_hi: float, mode: int) -> None:
    _check_f32('i_var', i_var), _check_f32('fb', fb)
    m = i_var.numel()
    _need(amax.numel() == m * n_parts and amax.dtype == torch.int32 and amax.is_cuda,
          'amax must be an int32 GPU tensor of n_parts slices matching i_var')
    _need(fb.numel() == m, 'fb must match i_var')
    if k_var.numel():
        _need(k_var.dtype == torch.uint8 and k_var.numel() == m and anyneg.numel() == m * n_parts,
              'k_var must be uint8 matching i_var')
    rc = _lib.load().hgq_wrap_track_i(_ptr(amax), _ptr(anyneg), n_parts, _ptr(i_var), _ptr(fb), _ptr(k_var), m, decay,
                                      c_lo, c_hi, mode, _stream())
    _lib.check(rc, 'hgq_wrap_track_i')


class _TrackItem(ctypes.Structure):
    _fields_ = [('amax', ctypes.c_void_p), ('anyneg', ctypes.c_void_p), ('n_parts', ctypes.c_int32), ('i_var', ctypes.c_void_p),
                ('fb', ctypes.c_void_p), ('k_var', ctypes.c_void_p), ('m', ctypes.c_int64), ('decay', ctypes.c_float),
                ('c_lo', ctypes.c_float), ('c_hi', ctypes.c_float), ('mode', ctypes.c_int32)]


@torch.library.custom_op('hgq::wrap_track_i_multi', mutates_args=('i_vars',))
def wrap_track_i_multi_op(amaxs: Sequence[Tensor], i_vars: Sequence[Tensor], fbs: Sequence[Tensor], decays: Sequence[float],
                          modes: Sequence[int]) -> None:
    """The training-mode integer-bit update of several quantizers (no sign tracker, no constraint) in one launch."""
    n = len(i_vars)
    items = (_TrackItem * n)()
    for t in range(n):
        _check_f32('i_var', i_vars[t]), _check_f32('fb', fbs[t])
        m = i_vars[t].numel()
        _need(m > 0 and amaxs[t].numel() % m == 0 and amaxs[t].numel() >= m and amaxs[t].dtype == torch.int32 and amaxs[t].is_cuda,
              'amax must be an int32 GPU tensor of whole slices matching i_var')
        _need(fbs[t].numel() == m, 'fb must match i_var')
        items[t] = _TrackItem(amaxs[t].data_ptr(), None, amaxs[t].numel() // m, i_vars[t].data_ptr(), fbs[t].data_ptr(), None, m,
                              decays[t], 0.0, 0.0, modes[t])
    rc = _lib.load().hgq_wrap_track_i_multi(items, n, _stream())
    _lib.check(rc, 'hgq_wrap_track_i_multi')


@torch.library.custom_op('hgq::qdense_fwd', mutates_args=())
def qdense_fwd(x: Tensor, k_in: Tensor, i_in: Tensor, f_in: Tensor, qw: Tensor, qb: Tensor, act: int, mode: int,
               bw_rows: int, track: bool) -> tuple[Tensor, Tensor]:
    _check_f32('x', x), _check_f32('qw', qw)
    _need(x.dim() == 2 and qw.dim() == 2 and x.shape[1] == qw.shape[0], f'shape mismatch {tuple(x.shape)} @ {tuple(qw.shape)}')
    rows, K = x.shape
    N = qw.shape[1]
    if qb.numel():
        _check_f32('qb', qb)
        _need(qb.numel() == N, 'bias size mismatch')
    if bw_rows > 0:
        _check_k('k_in', k_in), _check_f32('i_in', i_in), _check_f32('f_in', f_in)
        _need(i_in.numel() == bw_rows * K and f_in.numel() == bw_rows * K and k_in.numel() == bw_rows * K,
              'input bit-widths must have bw_rows*K elements')
        _need(rows % bw_rows == 0, 'rows must be a multiple of bw_rows')
        mode = _kmode(mode, k_in)
    lib = _lib.load()
    y = torch.empty((rows, N), dtype=torch.float32, device=x.device)
    if track and bw_rows > 0:
        amax = torch.empty((lib.hgq_qdense_fwd_parts(rows), bw_rows * K), dtype=torch.int32, device=x.device)
    else:
        amax = torch.empty((0, 0), dtype=torch.int32, device=x.device)
    rc = lib.hgq_qdense_fwd(_ptr(x), _ptr(k_in), _ptr(i_in), _ptr(f_in), bw_rows, _ptr(qw), _ptr(qb), _ptr(y), _ptr(amax),
                            rows, K, N, act, mode, _stream())
    _lib.check(rc, 'hgq_qdense_fwd')
    return y, amax


@qdense_fwd.register_fake
def _(x, k_in, i_in, f_in, qw, qb, act, mode, bw_rows, track):
    return x.new_empty((x.shape[0], qw.shape[1])), x.new_empty((0, 0), dtype=torch.int32)


@torch.library.custom_op('hgq::qdense_fwd_oq', mutates_args=())
def qdense_fwd_oq(x: Tensor, k_in: Tensor, f_in: Tensor, qw: Tensor, qb: Tensor, k_out: Tensor, f_out: Tensor, act: int,
                  mode: int, mode_out: int, bw_rows: int, bw_rows_out: int) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    """``qdense_fwd`` with the output quantizer on the tile as it leaves: ``(y, q_out(y), amax slices of the input
    quantizer, amax slices of the output quantizer)``."""
    _check_f32('x', x), _check_f32('qw', qw), _check_f32('f_in', f_in), _check_f32('f_out', f_out)
    _need(x.dim() == 2 and qw.dim() == 2 and x.shape[1] == qw.shape[0], f'shape mismatch {tuple(x.shape)} @ {tuple(qw.shape)}')
    rows, K = x.shape
    N = qw.shape[1]
    if qb.numel():
        _check_f32('qb', qb)
        _need(qb.numel() == N, 'bias size mismatch')
    _need(f_in.numel() == bw_rows * K and f_out.numel() == bw_rows_out * N, 'fractional-bit tables must be [bw_rows, K] and [bw_rows_out, N]')
    mode, mode_out = _kmode(mode, k_in), _kmode(mode_out, k_out)
    lib = _lib.load()
    y, yq = torch.empty((rows, N), dtype=torch.float32, device=x.device), torch.empty((rows, N), dtype=torch.float32, device=x.device)
    parts = lib.hgq_qdense_fwd_parts(rows)
    amax = torch.empty((parts, bw_rows * K), dtype=torch.int32, device=x.device)
    oamax = torch.empty((parts, bw_rows_out * N), dtype=torch.int32, device=x.device)
    rc = lib.hgq_qdense_fwd_oq(_ptr(x), _ptr(f_in), bw_rows, _ptr(qw), _ptr(qb), _ptr(f_out), bw_rows_out, _ptr(y), _ptr(yq), _ptr(amax),
                               _ptr(oamax), rows, K, N, act, mode, mode_out, _stream())
    _lib.check(rc, 'hgq_qdense_fwd_oq')
    return y, yq, amax, oamax


@qdense_fwd_oq.register_fake
def _(x, k_in, f_in, qw, qb, k_out, f_out, act, mode, mode_out, bw_rows, bw_rows_out):
    rows, N = x.shape[0], qw.shape[1]
    return (x.new_empty((rows, N)), x.new_empty((rows, N)), x.new_empty((1, f_in.numel()), dtype=torch.int32),
            x.new_empty((1, f_out.numel()), dtype=torch.int32))


@torch.library.custom_op('hgq::qdense_bwd', mutates_args=())
def qdense_bwd(dy: Tensor, y: Tensor, x: Tensor, f_in: Tensor, qw: Tensor, has_bias: bool, act: int, mode: int,
               bw_rows: int) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    _check_f32('dy', dy), _check_f32('x', x), _check_f32('qw', qw), _check_f32('y', y)
    rows, K = x.shape
    N = qw.shape[1]
    _need(tuple(dy.shape) == (rows, N), 'dy shape mismatch')
    lib = _lib.load()
    dx = torch.empty_like(x)
    dqw = torch.empty_like(qw)
    dqb = torch.empty(N if has_bias else 0, dtype=torch.float32, device=x.device)
    df = torch.empty(bw_rows * K, dtype=torch.float32, device=x.device)
    ws = torch.empty(lib.hgq_qdense_bwd_workspace(rows, K, N, bw_rows), dtype=torch.float32, device=x.device)
    rc = lib.hgq_qdense_bwd(_ptr(dy), _ptr(y), _ptr(x), _ptr(f_in), bw_rows, _ptr(qw), _ptr(dx), _ptr(dqw), _ptr(dqb),
                            _ptr(df), _ptr(ws), rows, K, N, act, mode, _stream())
    _lib.check(rc, 'hgq_qdense_bwd')
    return dx, dqw, dqb, df


@qdense_bwd.register_fake
def _(dy, y, x, f_in, qw, has_bias, act, mode, bw_rows):
    return (torch.empty_like(x), torch.empty_like(qw), x.new_empty(qw.shape[1] if has_bias else 0),
            x.new_empty(bw_rows * x.shape[1]))


@torch.library.custom_op('hgq::qdense_bwd_slices', mutates_args=())
def qdense_bwd_slices(dy: Tensor, y: Tensor, x: Tensor, f_in: Tensor, qw: Tensor, has_bias: bool, act: int, mode: int,
                      bw_rows: int) -> tuple[Tensor, Tensor]:
    """The dense backward without its slice reduction: ``(dx, slices [n, K*N + N + bw_rows*K])``."""
    _check_f32('dy', dy), _check_f32('x', x), _check_f32('qw', qw), _check_f32('y', y)
    rows, K = x.shape
    N = qw.shape[1]
    _need(tuple(dy.shape) == (rows, N), 'dy shape mismatch')
    lib = _lib.load()
    dx = torch.empty_like(x)
    width = K * N + N + bw_rows * K
    ws = torch.empty((lib.hgq_qdense_bwd_workspace(rows, K, N, bw_rows) // width, width), dtype=torch.float32, device=x.device)
    rc = lib.hgq_qdense_bwd_slices(_ptr(dy), _ptr(y), _ptr(x), _ptr(f_in), bw_rows, _ptr(qw), _ptr(dx), _ptr(ws), int(has_bias), rows, K, N,
                                   act, mode, _stream())
    _lib.check(rc, 'hgq_qdense_bwd_slices')
    return dx, ws


@qdense_bwd_slices.register_fake
def _(dy, y, x, f_in, qw, has_bias, act, mode, bw_rows):
    K, N = x.shape[1], qw.shape[1]
    return torch.empty_like(x), x.new_empty((max(1, -(-x.shape[0] // 64)), K * N + N + bw_rows * K))


def _check_relu_mask(mask: Tensor, rows: int, act: int) -> None:
    if act == _lib.ACT_RELU:
        _need(mask.is_cuda and mask.dtype == torch.int32 and mask.is_contiguous() and tuple(mask.shape) == (rows, 2),
              'the ReLU mask must be the [rows, 2] int32 tensor the forward pass left')


@torch.library.custom_op('hgq::qdense_fwd_mean', mutates_args=())
def qdense_fwd_mean(x: Tensor, k_in: Tensor, f_in: Tensor, qw: Tensor, qb: Tensor, act: int, mode: int, bw_rows: int,
                    mean_rows: int) -> tuple[Tensor, Tensor, Tensor]:
    """``qdense_fwd`` and the mean over groups of ``mean_rows`` consecutive output rows in one launch; the output itself is not
    written: ``(ReLU mask [rows, 2] - a bit per output, empty without ReLU -, group means [rows / mean_rows, N], amax slices of
    the input quantizer)``."""
    _check_f32('x', x), _check_f32('qw', qw)
    _need(x.dim() == 2 and qw.dim() == 2 and x.shape[1] == qw.shape[0], f'shape mismatch {tuple(x.shape)} @ {tuple(qw.shape)}')
    rows, K = x.shape
    N = qw.shape[1]
    if qb.numel():
        _check_f32('qb', qb)
        _need(qb.numel() == N, 'bias size mismatch')
    if bw_rows > 0:
        _check_f32('f_in', f_in)
        _need(f_in.numel() == bw_rows * K, 'the fractional-bit table must be [bw_rows, K]')
        mode = _kmode(mode, k_in)
    _need(mean_rows > 0 and rows % mean_rows == 0, 'rows must be a multiple of mean_rows')
    lib = _lib.load()
    mask = torch.empty((rows if act == _lib.ACT_RELU else 0, 2), dtype=torch.int32, device=x.device)
    ymean = torch.empty((rows // mean_rows, N), dtype=torch.float32, device=x.device)
    amax = torch.empty((lib.hgq_qdense_fwd_parts(rows) if bw_rows > 0 else 0, bw_rows * K), dtype=torch.int32, device=x.device)
    rc = lib.hgq_qdense_fwd_mean(_ptr(x), _ptr(f_in), bw_rows, _ptr(qw), _ptr(qb), _ptr(mask), _ptr(ymean), _ptr(amax), rows, K, N, mean_rows,
                                 act, mode, _stream())
    _lib.check(rc, 'hgq_qdense_fwd_mean')
    return mask, ymean, amax


@qdense_fwd_mean.register_fake
def _(x, k_in, f_in, qw, qb, act, mode, bw_rows, mean_rows):
    rows, N = x.shape[0], qw.shape[1]
    return (x.new_empty((rows if act == _lib.ACT_RELU else 0, 2), dtype=torch.int32), x.new_empty((rows // mean_rows, N)),
            x.new_empty((1 if bw_rows > 0 else 0, f_in.numel()), dtype=torch.int32))


@torch.library.custom_op('hgq::qdense_bwd_mean', mutates_args=())
def qdense_bwd_mean(dmean: Tensor, mask: Tensor, x: Tensor, f_in: Tensor, qw: Tensor, has_bias: bool, act: int, mode: int,
                    bw_rows: int, mean_rows: int) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    """``qdense_bwd`` from the gradient of the group means ``dmean`` [rows / mean_rows, N] and the forward's ReLU mask."""
    _check_f32('dmean', dmean), _check_f32('x', x), _check_f32('qw', qw)
    rows, K = x.shape
    N = qw.shape[1]
    _need(mean_rows > 0 and rows % mean_rows == 0 and tuple(dmean.shape) == (rows // mean_rows, N), 'dmean shape mismatch')
    _check_relu_mask(mask, rows, act)
    lib = _lib.load()
    dx = torch.empty_like(x)
    dqw = torch.empty_like(qw)
    dqb = torch.empty(N if has_bias else 0, dtype=torch.float32, device=x.device)
    df = torch.empty(bw_rows * K, dtype=torch.float32, device=x.device)
    ws = torch.empty(lib.hgq_qdense_bwd_workspace(rows, K, N, bw_rows), dtype=torch.float32, device=x.device)
    rc = lib.hgq_qdense_bwd_mean(_ptr(dmean), _ptr(mask), _ptr(x), _ptr(f_in), bw_rows, _ptr(qw), _ptr(dx), _ptr(dqw), _ptr(dqb), _ptr(df),
                                 _ptr(ws), rows, K, N, mean_rows, act, mode, _stream())
    _lib.check(rc, 'hgq_qdense_bwd_mean')
    return dx, dqw, dqb, df


@qdense_bwd_mean.register_fake
def _(dmean, mask, x, f_in, qw, has_bias, act, mode, bw_rows, mean_rows):
    return (torch.empty_like(x), torch.empty_like(qw), x.new_empty(qw.shape[1] if has_bias else 0),
            x.new_empty(bw_rows * x.shape[1]))


@torch.library.custom_op('hgq::qdense_bwd_mean_slices', mutates_args=())
def qdense_bwd_mean_slices(dmean: Tensor, mask: Tensor, x: Tensor, f_in: Tensor, qw: Tensor, has_bias: bool, act: int, mode: int,
                           bw_rows: int, mean_rows: int) -> tuple[Tensor, Tensor]:
    """``qdense_bwd_slices`` from the gradient of the group means ``dmean`` [rows / mean_rows, N] and the forward's ReLU mask."""
    _check_f32('dmean', dmean), _check_f32('x', x), _check_f32('qw', qw)
    rows, K = x.shape
    N = qw.shape[1]
    _need(mean_rows > 0 and rows % mean_rows == 0 and tuple(dmean.shape) == (rows // mean_rows, N), 'dmean shape mismatch')
    _check_relu_mask(mask, rows, act)
    lib = _lib.load()
    dx = torch.empty_like(x)
    width = K * N + N + bw_rows * K
    ws = torch.empty((lib.hgq_qdense_bwd_workspace(rows, K, N, bw_rows) // width, width), dtype=torch.float32, device=x.device)
    rc = lib.hgq_qdense_bwd_mean_slices(_ptr(dmean), _ptr(mask), _ptr(x), _ptr(f_in), bw_rows, _ptr(qw), _ptr(dx), _ptr(ws), int(has_bias), rows,
                                        K, N, mean_rows, act, mode, _stream())
    _lib.check(rc, 'hgq_qdense_bwd_mean_slices')
    return dx, ws


@qdense_bwd_mean_slices.register_fake
def _(dmean, mask, x, f_in, qw, has_bias, act, mode, bw_rows, mean_rows):
    K, N = x.shape[1], qw.shape[1]
    return torch.empty_like(x), x.new_empty((max(1, -(-x.shape[0] // 64)), K * N + N + bw_rows * K))


class _ReduceItem(ctypes.Structure):
    _fields_ = [('slices', ctypes.c_void_p), ('n_slices', ctypes.c_int32), ('width', ctypes.c_int64), ('out', ctypes.c_void_p * 3),
                ('n_out', ctypes.c_int64 * 3)]


@torch.library.custom_op('hgq::reduce_slices_multi', mutates_args=('outs',))
def reduce_slices_multi_op(slices: Sequence[Tensor], outs: Sequence[Tensor], skip: Sequence[bool]) -> None:
    """``outs[3t .. 3t+2]`` (concatenated) = column sums of ``slices[t]`` [n, width], fixed order, all sets in one launch; a
    segment with ``skip`` set has its length in ``outs`` but is not written."""
    items = _reduce_items(slices, outs, skip)
    rc = _lib.load().hgq_reduce_slices_multi(items, len(slices), _stream())
    _lib.check(rc, 'hgq_reduce_slices_multi')


def _reduce_items(slices, outs, skip):
    n = len(slices)
    _need(len(outs) == 3 * n and len(skip) == 3 * n, 'three outputs per slice set')
    items = (_ReduceItem * max(n, 1))()
    for t in range(n):
        sl = slices[t]
        _check_f32('slices', sl)
        _need(sl.dim() == 2 and sl.shape[0] >= 1, 'slices must be [n, width]')
        o = outs[3 * t:3 * t + 3]
        for v in o:
            _check_f32('out', v)
        _need(sum(v.numel() for v in o) == sl.shape[1], 'outputs do not add up to the slice width')
        items[t].slices, items[t].n_slices, items[t].width = sl.data_ptr(), sl.shape[0], sl.shape[1]
        for j in range(3):
            items[t].out[j] = o[j].data_ptr() if (o[j].numel() and not skip[3 * t + j]) else None
            items[t].n_out[j] = o[j].numel()
    return items


REDUCE_BATCH, REDUCE_QUANTS = 16, 24  # HGQ_REDUCE_BATCH, HGQ_REDUCE_QUANTS


@torch.library.custom_op('hgq::reduce_slices_quant_multi', mutates_args=('outs',))
def reduce_slices_quant_multi_op(slices: Sequence[Tensor], outs: Sequence[Tensor], skip: Sequence[bool], xs: Sequence[Tensor],
                                 ks: Sequence[Tensor], is_: Sequence[Tensor], fbs: Sequence[Tensor], modes: Sequence[int],
                                 q_set: Sequence[int], q_segment: Sequence[int]) -> list[Tensor]:
    """``reduce_slices_multi_op`` with the backward of quantizers whose upstream gradient is a reduced segment run on the
    sums as they are formed: quantizer j (per-element bit-widths) reads segment ``q_segment[j]`` of slice set ``q_set[j]``.
    Returns ``dx_0 .., di_0 .., dfb_0 ..`` as ``quantize_bwd_multi`` does."""
    items = _reduce_items(slices, outs, skip)
    _check_multi(xs, ks, is_, fbs, modes)
    n = len(xs)
    _need(len(q_set) == n and len(q_segment) == n, 'one slice set and segment per quantizer')
    dxs, dis, dfs = [torch.empty_like(x) for x in xs], [torch.empty_like(i) for i in is_], [torch.empty_like(f) for f in fbs]
    quants = (_QuantGradItem * max(n, 1))()
    for t in range(n):
        quants[t] = _QuantGradItem(0, xs[t].data_ptr(), ks[t].data_ptr(), is_[t].data_ptr(), fbs[t].data_ptr(), dxs[t].data_ptr(),
                                   dis[t].data_ptr(), dfs[t].data_ptr(), xs[t].numel(), _kmode(modes[t], ks[t]))
    sets, segs = (ctypes.c_int * max(n, 1))(*q_set), (ctypes.c_int * max(n, 1))(*q_segment)
    rc = _lib.load().hgq_reduce_slices_quant_multi(items, len(slices), quants, sets, segs, n, _stream())
    _lib.check(rc, 'hgq_reduce_slices_quant_multi')
    return dxs + dis + dfs


@reduce_slices_quant_multi_op.register_fake
def _(slices, outs, skip, xs, ks, is_, fbs, modes, q_set, q_segment):
    return [torch.empty_like(x) for x in xs] + [torch.empty_like(i) for i in is_] + [torch.empty_like(f) for f in fbs]


# ---- slice reductions whose results nothing reads before the kernel / bias quantizers' backward or the optimizer:
# queued while the gradient sink is open, run as one launch by ``flush_reductions``
_PENDING_REDUCE: list = []


def flush_reductions():
    if not _PENDING_REDUCE:
        return
    sl, outs, skip = [], [], []
    for s_, o_, k_ in _PENDING_REDUCE:
        sl.append(s_), outs.extend(o_), skip.extend(k_)
    _PENDING_REDUCE.clear()
    reduce_slices_multi_op(sl, outs, skip)


def _reduce_and_quantize_bwd(dys, xs, ks, is_, fbs, modes):
    """The pending slice reductions and the backward of the quantizers ``xs`` in ONE launch, when every upstream gradient in
    ``dys`` is a whole segment of a pending reduction (the kernel / bias gradients a contraction's backward left as slices):
    the quantizer backward then runs on the sums as they are formed.  Returns what ``quantize_bwd_multi`` returns, or ``None``
    when the gradients come from elsewhere (the caller flushes and launches the two separately)."""
    if not _PENDING_REDUCE or not dys or len(dys) > REDUCE_QUANTS or len(_PENDING_REDUCE) > REDUCE_BATCH:
        return None
    where = {}
    for t, (_, outs, _) in enumerate(_PENDING_REDUCE):
        for seg, o in enumerate(outs):
            if o.numel():
                where[(o.data_ptr(), o.numel())] = (t, seg)
    q_set, q_seg = [], []
    for dy, x in zip(dys, xs):
        hit = where.pop((dy.data_ptr(), dy.numel()), None) if dy.numel() == x.numel() and dy.numel() else None
        if hit is None:
            return None
        q_set.append(hit[0]), q_seg.append(hit[1])
    sl, outs, skip = [], [], []
    for s_, o_, k_ in _PENDING_REDUCE:
        sl.append(s_), outs.extend(o_), skip.extend(k_)
    for t, seg in zip(q_set, q_seg):
        skip[3 * t + seg] = True  # read by the quantizer's backward inside the launch and by nothing else
    _PENDING_REDUCE.clear()
    return reduce_slices_quant_multi_op(sl, outs, skip, list(xs), list(ks), list(is_), list(fbs), list(modes), q_set, q_seg)


def _dense_ebops_check(amax, beta, k_in, i_in, f_in, k_ker, b_ker, k_bias, b_bias, ebops_var, P, K, N, mode_in, mode_ker, mode_bias):
    """Validates one dense-EBOPs call; returns ``(n_parts, has_bias, mode_in, mode_ker, mode_bias)`` with the k-storage flags set."""
    _check_k('k_in', k_in), _check_f32('i_in', i_in), _check_f32('f_in', f_in), _check_k('k_ker', k_ker), _check_f32('b_ker', b_ker)
    _need(i_in.numel() == P * K and f_in.numel() == P * K and k_in.numel() == P * K, 'input bit-width size mismatch')
    _need(b_ker.numel() == K * N and k_ker.numel() == K * N, 'kernel bit-width size mismatch')
    has_bias = b_bias.numel() > 0
    if has_bias:
        _check_f32('b_bias', b_bias), _check_k('k_bias', k_bias)
        _need(b_bias.numel() == N and k_bias.numel() == N, 'bias bit-width size mismatch')
        mode_bias = _kmode(mode_bias, k_bias)
    n_parts = 0
    if amax.numel():
        _need(amax.dtype == torch.int32 and amax.is_cuda and amax.numel() % (P * K) == 0, 'amax slices must be [n_parts, P*K] int32')
        n_parts = amax.numel() // (P * K)
    if ebops_var.numel():
        _need(ebops_var.is_cuda and ebops_var.element_size() == 4, 'the ebops variable must be a 4-byte GPU scalar')
    if beta.numel():
        _check_f32('beta', beta)
    return n_parts, has_bias, _kmode(mode_in, k_in), _kmode(mode_ker, k_ker), mode_bias


def _dense_ebops_impl(amax: Tensor, decay: float, beta: Tensor, k_in: Tensor, i_in: Tensor, f_in: Tensor, k_ker: Tensor,
                   b_ker: Tensor, k_bias: Tensor, b_bias: Tensor, ebops_var: Tensor, P: int, K: int, N: int, par_factor: float,
                   n_parallel: float, ebops_factor: float, bias_size: float, mode_in: int, mode_ker: int, mode_bias: int) -> tuple[Tensor, Tensor, Tensor]:
    """Returns (ebops, ebops*beta, [g_f_in | g_b_ker | g_b_bias] in one buffer); with ``beta`` the
    gradient buffer holds d(ebops*beta)/d variable, else d ebops / d variable."""
    n_parts, has_bias, m_in, m_ker, m_bias = _dense_ebops_check(amax, beta, k_in, i_in, f_in, k_ker, b_ker, k_bias, b_bias, ebops_var,
                                                               P, K, N, mode_in, mode_ker, mode_bias)
    dev = f_in.device
    ebops = torch.empty((), dtype=torch.float32, device=dev)
    term = torch.empty((), dtype=torch.float32, device=dev)
    nb = N if has_bias else 0
    g = torch.empty(P * K + K * N + nb, dtype=torch.float32, device=dev)
    g_f, g_bk, g_bb = g[:P * K], g[P * K:P * K + K * N], g[P * K + K * N:]
    rc = _lib.load().hgq_dense_ebops(_ptr(amax), n_parts, decay, _ptr(beta), _ptr(term), _ptr(k_in), _ptr(i_in), _ptr(f_in),
                                     P, K, N, _ptr(k_ker), _ptr(b_ker), _ptr(k_bias), _ptr(b_bias), par_factor, n_parallel, ebops_factor, bias_size,
                                     m_in, m_ker, m_bias, _ptr(ebops), _ptr(ebops_var),
                                     _ptr(g_f), _ptr(g_bk), _ptr(g_bb), _stream())
    _lib.check(rc, 'hgq_dense_ebops')
    return ebops, term, g


class _DenseEbopsItem(ctypes.Structure):
    _fields_ = [('amax_part', ctypes.c_void_p), ('n_parts', ctypes.c_int), ('decay', ctypes.c_float), ('beta', ctypes.c_void_p),
                ('loss_term', ctypes.c_void_p), ('k_in', ctypes.c_void_p), ('i_in', ctypes.c_void_p), ('f_in', ctypes.c_void_p),
                ('P', ctypes.c_int64), ('K', ctypes.c_int), ('N', ctypes.c_int), ('k_ker', ctypes.c_void_p), ('b_ker', ctypes.c_void_p),
                ('k_bias', ctypes.c_void_p), ('b_bias', ctypes.c_void_p), ('par_factor', ctypes.c_float), ('n_parallel', ctypes.c_float), ('ebops_factor', ctypes.c_float),
                ('bias_size', ctypes.c_float),
                ('mode_in', ctypes.c_int), ('mode_ker', ctypes.c_int), ('mode_bias', ctypes.c_int), ('ebops', ctypes.c_void_p),
                ('ebops_u32', ctypes.c_void_p), ('g_f_in', ctypes.c_void_p), ('g_b_ker', ctypes.c_void_p), ('g_b_bias', ctypes.c_void_p)]


@torch.library.custom_op('hgq::dense_ebops_multi', mutates_args=('i_ins', 'ebops_vars', 'ebops_outs', 'terms', 'gs'))
def dense_ebops_multi_op(amaxs: Sequence[Tensor], betas: Sequence[Tensor], k_ins: Sequence[Tensor], i_ins: Sequence[Tensor],
                         f_ins: Sequence[Tensor], k_kers: Sequence[Tensor], b_kers: Sequence[Tensor], k_biases: Sequence[Tensor],
                         b_biases: Sequence[Tensor], ebops_vars: Sequence[Tensor], ebops_outs: Sequence[Tensor], terms: Sequence[Tensor],
                         gs: Sequence[Tensor], decays: Sequence[float], dims: Sequence[int], scales: Sequence[float],
                         bias_sizes: Sequence[float], modes: Sequence[int]) -> None:
    """The dense-EBOPs launch of several layers at once; outputs are preallocated (``ebops_outs``, ``terms``, ``gs`` as
    ``_dense_ebops_impl`` returns them).  ``dims`` = P, K, N per item, ``scales`` = par_factor, n_parallel, ebops_factor per item,
    ``modes`` = mode_in, mode_ker, mode_bias per item."""
    n = len(f_ins)
    items = (_DenseEbopsItem * n)()
    for t in range(n):
        P, K, N = dims[3 * t:3 * t + 3]
        n_parts, has_bias, m_in, m_ker, m_bias = _dense_ebops_check(
            amaxs[t], betas[t], k_ins[t], i_ins[t], f_ins[t], k_kers[t], b_kers[t], k_biases[t], b_biases[t], ebops_vars[t], P, K, N,
            modes[3 * t], modes[3 * t + 1], modes[3 * t + 2])
        g = gs[t]
        _need(g.numel() == P * K + K * N + (N if has_bias else 0) and g.is_contiguous(), 'gradient buffer size mismatch')
        g_f, g_bk, g_bb = g[:P * K], g[P * K:P * K + K * N], g[P * K + K * N:]
        p = lambda x: x.data_ptr() if x.numel() else None  # noqa: E731
        items[t] = _DenseEbopsItem(p(amaxs[t]), n_parts, decays[t], p(betas[t]), p(terms[t]), p(k_ins[t]), p(i_ins[t]), p(f_ins[t]), P, K, N,
                                   p(k_kers[t]), p(b_kers[t]), p(k_biases[t]), p(b_biases[t]), scales[3 * t], scales[3 * t + 1], scales[3 * t + 2], bias_sizes[t], m_in, m_ker, m_bias,
                                   p(ebops_outs[t]), p(ebops_vars[t]), p(g_f), p(g_bk), p(g_bb))
    rc = _lib.load().hgq_dense_ebops_multi(items, n, _stream())
    _lib.check(rc, 'hgq_dense_ebops_multi')


# ---- state epoch: bumped by everything in this package that writes variables through `.data` or from a kernel (writes
# the tensors' version counters do not see); a cache keyed on variable versions also keys on it
STATE_EPOCH = [0]


def touch_state():
    STATE_EPOCH[0] += 1


# ---- launches on a second stream
# The EBOPs estimates read bit-width variables (and the abs-max slices a quantizer left); what they write - the loss
# term, the uint32 variable, gradient pieces - is read again only when the loss is summed and when the optimizer
# steps.  They are single-workgroup, latency-bound launches.  Inside ``overlap_ebops()`` they go to a second stream
# (default priority) that forks from the current one where they are issued and is joined where their results are read,
# so they run beside the layers' data kernels; in a captured step the fork and join become edges of the graph.
_OVERLAP = {'depth': 0, 'streams': {}, 'pending': [], 'keep': [], 'finish': []}


class overlap_ebops:
    """Context manager around a training step (forward, loss, backward, update): EBOPs launches inside it run on a
    second stream.  Whoever opens it must leave it before the captured graph ends or before results are read from
    another thread or stream; leaving it joins the second stream.  ``hgq2_amd.train.model_loss`` called inside it
    returns a total whose value is there once the context is left (its gradient does not need the value)."""

    def __enter__(self):
        _claim_step('overlap_ebops')
        _OVERLAP['depth'] += 1
        return self

    def __exit__(self, *exc):
        _OVERLAP['depth'] -= 1
        try:
            if _OVERLAP['depth'] == 0:
                join_side()
        finally:
            _release_step()
        return False


class side_branch:
    """The launches inside go to the second stream when ``overlap_ebops`` is open (else nothing changes)."""

    def __enter__(self):
        self.ctx = None
        if _OVERLAP['depth'] and torch.cuda.is_available():
            cur = torch.cuda.current_stream()
            side = _OVERLAP['streams'].get(cur.device)
            if side is None:
                side = _OVERLAP['streams'][cur.device] = torch.cuda.Stream(device=cur.device)
            if side != cur:
                side.wait_stream(cur)  # everything issued so far is visible to the branch
                if not any(s is side for _, s in _OVERLAP['pending']):
                    _OVERLAP['pending'].append((cur, side))
                self.ctx = torch.cuda.stream(side)
                self.ctx.__enter__()
        return self

    def __exit__(self, *exc):
        if self.ctx is not None:
            self.ctx.__exit__(*exc)
        return False


def join_side(hand_over_sums: bool = False, sums_later: bool = False):
    """The current stream waits for the second stream's work (no-op when there is none).  Work that needed both streams'
    results - the sums of loss terms, ``(terms, out)`` pairs - runs now, or is returned to a caller that folds it into a
    launch of its own (``hand_over_sums``; sums of more than ``SUM_BATCH`` terms run here either way), or stays queued
    for the next join (``sums_later``: a join in the middle of a step; the one that ends the step finds them)."""
    pending, _OVERLAP['pending'] = _OVERLAP['pending'], []
    for cur, side in pending:
        torch.cuda.current_stream(cur.device).wait_stream(side)
    if sums_later:
        return []
    finish, _OVERLAP['finish'] = _OVERLAP['finish'], []
    handed = []
    for terms, out in finish:
        if hand_over_sums and len(terms) <= SUM_BATCH:
            handed.append((terms, out))
        else:
            sum_scalars_into(terms, out)
    _OVERLAP['keep'] = []
    return handed


def _keep(tensors):
    """Short-lived inputs of a launch that may be on the second stream (tracker slices written by the data kernels) stay
    referenced until the streams are joined: the allocator would otherwise hand their memory to a later launch of the
    first stream while the second still reads it."""
    if _OVERLAP['depth']:
        _OVERLAP['keep'].extend(t for t in tensors if t is not None)


# ---- launches deferred to the end of the outermost layer call
# The EBOPs estimate of a dense layer (and the integer-bit update fused into it) reads bit-width variables and the
# abs-max slices its own forward left; nothing later in the forward pass reads what it writes.  While a model call is
# open the calls are queued - outputs allocated, nothing launched - and go out as one launch when the call returns.
_DEFER = {'depth': 0, 'dense_ebops': [], 'tracks': [], 'late': []}


def begin_deferred():
    _claim_step('model call')
    _DEFER['depth'] += 1


def end_deferred(discard: bool = False):
    _DEFER['depth'] -= 1
    try:
        if _DEFER['depth'] == 0:
            if discard:
                _DEFER['dense_ebops'], _DEFER['tracks'], _DEFER['late'] = [], [], []
            elif _OVERLAP['depth'] and _worth_a_branch():
                with side_branch():
                    flush_deferred()
            else:
                flush_deferred()
    finally:
        _release_step()


def _rounds(keys):
    """Split queue positions into launches: entries of one launch run concurrently, so entries with the same key (the
    address of the integer-bit variable they update or read) go to successive launches, in queue order.  A quantizer
    shared by several layers (the fused inputs of an attention layer, reference src/hgq/layers/attn/mha.py:205-210) is
    updated once per call of each layer, one after the other."""
    rounds, seen = [], {}
    for n, key in enumerate(keys):
        r = seen.get(key, 0)
        seen[key] = r + 1
        if r == len(rounds):
            rounds.append([])
        rounds[r].append(n)
    return rounds


def _order_after_side():
    """A flush issued on the first stream while the second still has work of this step: the second goes first (its
    launches were queued earlier and may touch the same variables)."""
    if _OVERLAP['pending']:
        cur = torch.cuda.current_stream()
        if not any(cur == side for _, side in _OVERLAP['pending']):
            join_side(sums_later=True)


def flush_tracks():
    """Run the queued integer-bit updates (one launch; one more for every repeated update of the same variable).  Everything
    that reads integer bits of a WRAP quantizer inside a model call - the EBOPs launches, the bit-width views - calls
    this first."""
    q, _DEFER['tracks'] = _DEFER['tracks'], []
    if not q:
        return
    _order_after_side()
    touch_state()
    with torch.no_grad():
        _keep(item[0] for item in q)
        for members in _rounds([item[1].data_ptr() for item in q]):
            amaxs, i_vars, fbs, decays, modes = (list(c) for c in zip(*[q[n] for n in members]))
            wrap_track_i_multi_op(amaxs, i_vars, fbs, [float(d) for d in decays], [int(m) for m in modes])


def _reads_queued(i_var) -> bool:
    """Is a queued EBOPs launch going to read this integer-bit variable?"""
    ptr = i_var.data_ptr()
    return (any(item[3].data_ptr() == ptr for item in _DEFER['dense_ebops'])
            or any(ptr in reads for reads, _ in _DEFER['late']))


def _worth_a_branch() -> bool:
    """A fork and a join between two streams cost a replayed graph about 15 us of idle time on this platform, a queued
    single-workgroup launch hides 5 - 30 us: the branch pays from about three launches on, or one long one (the EBOPs of
    a contraction with a few thousand input channels)."""
    n = len(_DEFER['late']) + (1 if _DEFER['tracks'] else 0) + (1 if _DEFER['dense_ebops'] else 0)
    big = any(item[14][1] * item[14][2] >= 16384 for item in _DEFER['dense_ebops'])
    return n >= 3 or (big and n >= 2)


def flush_deferred():
    flush_tracks()
    if _DEFER['late'] or _DEFER['dense_ebops']:
        _order_after_side()
    late, _DEFER['late'] = _DEFER['late'], []
    _flush_dense_queue()
    for _, launch in late:
        launch()


def _flush_dense_queue():
    q, _DEFER['dense_ebops'] = _DEFER['dense_ebops'], []
    if not q:
        return
    touch_state()  # the fused integer-bit update writes `_i`
    with torch.no_grad():
        # inputs and outputs alike: an output nobody holds on to (the plain EBOPs value beside the loss term) would be
        # handed to the next allocation of the first stream and then overwritten from the second
        _keep(t for item in q for t in item if torch.is_tensor(t))
        # layers that share an input quantizer update and read its integer bits one after the other
        for members in _rounds([item[3].data_ptr() for item in q]):
            _flush_dense_ebops(*zip(*[q[n] for n in members]))


def _flush_dense_ebops(amaxs, betas, k_ins, i_ins, f_ins, k_kers, b_kers, k_biases, b_biases, ebops_vars, outs, terms, gs, decays, dims,
                       scales, bias_sizes, modes):
    dense_ebops_multi_op(list(amaxs), list(betas), list(k_ins), list(i_ins), list(f_ins), list(k_kers), list(b_kers), list(k_biases),
                         list(b_biases), list(ebops_vars), list(outs), list(terms), list(gs), [float(d) for d in decays],
                         [int(v) for d in dims for v in d], [float(v) for s in scales for v in s], [float(v) for v in bias_sizes],
                         [int(v) for m in modes for v in m])


def _dense_ebops_queue(amax, decay, beta, k_in, i_in, f_in, k_ker, b_ker, k_bias, b_bias, ebops_var, P, K, N, par_factor, n_parallel,
                       ebops_factor, bias_size,
                       mode_in, mode_ker, mode_bias):
    dev = f_in.device
    ebops = torch.empty((), dtype=torch.float32, device=dev)
    term = torch.empty((), dtype=torch.float32, device=dev)
    g = torch.empty(P * K + K * N + (N if b_bias.numel() else 0), dtype=torch.float32, device=dev)
    # `.data`: the update of the integer bits is a state assignment, not an operation autograd should see
    _DEFER['dense_ebops'].append((amax, beta, k_in, i_in.data, f_in, k_ker, b_ker, k_bias, b_bias, ebops_var, ebops, term, g, decay, (P, K, N),
                                  (par_factor, n_parallel, ebops_factor), bias_size, (mode_in, mode_ker, mode_bias)))
    return ebops, term, g


# Two registrations of the same launch: the tracking form updates the input quantizer's integer
# bits in place (and is declared so), the plain form leaves them alone.
dense_ebops_track_op = torch.library.custom_op('hgq::dense_ebops_track', _dense_ebops_impl, mutates_args=('i_in', 'ebops_var'))
dense_ebops_op = torch.library.custom_op('hgq::dense_ebops', _dense_ebops_impl, mutates_args=('ebops_var',))


_CE_STATE = {}


@torch.library.custom_op('hgq::sparse_ce', mutates_args=())
def sparse_ce_op(logits: Tensor, labels: Tensor) -> tuple[Tensor, Tensor]:
    _check_f32('logits', logits)
    _need(logits.dim() == 2 and labels.dim() == 1 and labels.shape[0] == logits.shape[0], 'logits [rows, C], labels [rows]')
    _need(labels.dtype == torch.int64 and labels.is_cuda and labels.is_contiguous(), 'labels must be a contiguous int64 GPU tensor')
    loss = torch.empty((), dtype=torch.float32, device=logits.device)
    dlogits = torch.empty_like(logits)
    # four words per (device, stream), zeroed once: the kernel leaves them zero, so no call clears anything
    stream = _stream()
    key = (logits.device, stream.value if hasattr(stream, 'value') else stream)
    state = _CE_STATE.get(key)
    if state is None:
        state = _CE_STATE[key] = torch.zeros(4, dtype=torch.int32, device=logits.device)
    rc = _lib.load().hgq_sparse_ce_fwd_bwd(_ptr(logits), _ptr(labels), _ptr(loss), _ptr(dlogits), logits.shape[0],
                                           logits.shape[1], _ptr(state), stream)
    _lib.check(rc, 'hgq_sparse_ce_fwd_bwd')
    return loss, dlogits


@sparse_ce_op.register_fake
def _(logits, labels):
    return logits.new_empty(()), torch.empty_like(logits)


@torch.library.custom_op('hgq::sgd_update', mutates_args=('w',))
def sgd_update_op(w: Tensor, g: Tensor, lr: float, l1: float, lo: float, hi: float) -> None:
    _check_f32('w', w), _check_f32('g', g)
    _need(w.numel() == g.numel(), 'gradient size mismatch')
    rc = _lib.load().hgq_sgd_update(_ptr(w), _ptr(g), w.numel(), lr, l1, lo, hi, _stream())
    _lib.check(rc, 'hgq_sgd_update')


SGD_SIDES = 4


class _SgdItem(ctypes.Structure):
    _fields_ = [('w', ctypes.c_void_p), ('g', ctypes.c_void_p), ('n', ctypes.c_int64), ('l1', ctypes.c_float),
                ('lo', ctypes.c_float), ('hi', ctypes.c_float), ('side', ctypes.c_void_p * SGD_SIDES),
                ('side_scale', ctypes.c_void_p * SGD_SIDES)]


@torch.library.custom_op('hgq::sgd_update_multi', mutates_args=('ws', 'sum_out'))
def sgd_update_multi_op(ws: Sequence[Tensor], gs: Sequence[Tensor], l1: Sequence[float], lo: Sequence[float],
                        hi: Sequence[float], lr: float, sides: Sequence[Tensor], side_scales: Sequence[Tensor],
                        sum_terms: Sequence[Tensor], sum_out: Tensor) -> None:
    """``gs[t]`` empty: no plain gradient.  ``sides`` / ``side_scales``: SGD_SIDES entries per variable (empty = absent;
    an absent scale means 1).  ``sum_terms`` (1 to SUM_BATCH one-element tensors, or none): added in list order into
    ``sum_out`` by the same launch - the step's loss terms, which the update does not read."""
    n = len(ws)
    _need(len(gs) == n and len(l1) == n and len(lo) == n and len(hi) == n, 'per-variable lists differ in length')
    _need(len(sides) == SGD_SIDES * n and len(side_scales) == SGD_SIDES * n, 'side-gradient lists must hold SGD_SIDES entries per variable')
    items = (_SgdItem * n)()
    for t, (w, g) in enumerate(zip(ws, gs)):
        _check_f32('w', w)
        if g.numel():
            _check_f32('g', g)
            _need(w.numel() == g.numel(), 'gradient size mismatch')
        it = _SgdItem(w.data_ptr(), g.data_ptr() if g.numel() else None, w.numel(), l1[t], lo[t], hi[t])
        for s in range(SGD_SIDES):
            sd, sc = sides[SGD_SIDES * t + s], side_scales[SGD_SIDES * t + s]
            if sd.numel():
                _check_f32('side gradient', sd)
                _need(sd.numel() == w.numel(), 'side gradient size mismatch')
                it.side[s] = sd.data_ptr()
                if sc.numel():
                    _need(sc.is_cuda and sc.dtype == torch.float32 and sc.numel() == 1, 'a side-gradient scale is one float32 on the GPU')
                    it.side_scale[s] = sc.data_ptr()
        items[t] = it
    if len(sum_terms):
        _need(len(sum_terms) <= SUM_BATCH, f'at most {SUM_BATCH} terms ride along with the update')
        ptrs = (ctypes.c_void_p * len(sum_terms))()
        for t, term in enumerate(sum_terms):
            _check_f32('term', term)
            _need(term.numel() == 1, 'every term must hold one element')
            ptrs[t] = term.data_ptr()
        _check_f32('sum_out', sum_out)
        rc = _lib.load().hgq_sgd_update_multi_sum(items, n, lr, ptrs, len(sum_terms), _ptr(sum_out), _stream())
        _lib.check(rc, 'hgq_sgd_update_multi_sum')
        return
    rc = _lib.load().hgq_sgd_update_multi(items, n, lr, _stream())
    _lib.check(rc, 'hgq_sgd_update_multi')


SUM_BATCH = 64


@torch.library.custom_op('hgq::sum_scalars', mutates_args=())
def sum_scalars_op(terms: Sequence[Tensor]) -> Tensor:
    n = len(terms)
    _need(1 <= n <= SUM_BATCH, f'1 to {SUM_BATCH} terms are expected')
    ptrs = (ctypes.c_void_p * n)()
    for t, term in enumerate(terms):
        _check_f32('term', term)
        _need(term.numel() == 1, 'every term must hold one element')
        ptrs[t] = term.data_ptr()
    out = torch.empty((), dtype=torch.float32, device=terms[0].device)
    rc = _lib.load().hgq_sum_scalars(ptrs, n, _ptr(out), _stream())
    _lib.check(rc, 'hgq_sum_scalars')
    return out


@sum_scalars_op.register_fake
def _(terms):
    return terms[0].new_empty(())


class _SumScalars(torch.autograd.Function):
    @staticmethod
    def forward(ctx, *terms):
        ctx.shapes = [t.shape for t in terms]
        return sum_scalars_op([t.detach() for t in terms])

    @staticmethod
    def backward(ctx, g):
        # every term receives the same upstream gradient: views of it, no launches
        return tuple(g.reshape(s) if ctx.needs_input_grad[t] else None for t, s in enumerate(ctx.shapes))


def sum_scalars_into(terms: Sequence[Tensor], out: Tensor) -> None:
    """``out <- ((terms[0] + terms[1]) + ...)`` (values only) on the current stream; ``out`` is a one-element fp32 GPU tensor."""
    terms = [t.detach() for t in terms]
    while len(terms) > SUM_BATCH:
        terms = [sum_scalars_op(terms[:SUM_BATCH])] + terms[SUM_BATCH:]
    n = len(terms)
    ptrs = (ctypes.c_void_p * n)()
    for t, term in enumerate(terms):
        _check_f32('term', term)
        _need(term.numel() == 1, 'every term must hold one element')
        ptrs[t] = term.data_ptr()
    _check_f32('out', out)
    rc = _lib.load().hgq_sum_scalars(ptrs, n, _ptr(out), _stream())
    _lib.check(rc, 'hgq_sum_scalars')


def sum_scalars(terms: Sequence[Tensor]) -> Tensor:
    """``((terms[0] + terms[1]) + terms[2]) + ...`` of one-element GPU tensors, in that order, in one launch
    (chunks of ``SUM_BATCH``); differentiable."""
    terms = list(terms)
    while len(terms) > 1:
        head, terms = terms[:SUM_BATCH], terms[SUM_BATCH:]
        terms.insert(0, _SumScalars.apply(*head))
    return terms[0]


def _qdescs(ks: Sequence[Tensor], is_: Sequence[Tensor], fbs: Sequence[Tensor], modes: Sequence[int]):
    """Five ``hgq_qdesc`` structures (exp_iq, exp_oq, inv_iq, inv_oq, oq); an empty ``k`` means absent."""
    _need(len(ks) == 5 and len(is_) == 5 and len(fbs) == 5 and len(modes) == 5, 'five quantizer descriptors are expected')
    descs = []
    for n, (k, i, fb, mode) in enumerate(zip(ks, is_, fbs, modes)):
        if k.numel() == 0:
            descs.append(_lib.QDesc(None, None, None, 0))
            continue
        _check_k(f'k[{n}]', k), _check_f32(f'i[{n}]', i), _check_f32(f'fb[{n}]', fb)
        _need(k.numel() == i.numel() == fb.numel(), f'quantizer {n}: k, i, fb differ in size')
        if n < 4:
            _need(i.numel() == 1, f'quantizer {n}: the table quantizers must have a single bit-width entry')
        descs.append(_lib.QDesc(k.data_ptr(), i.data_ptr(), fb.data_ptr(), _kmode(mode, k)))
    return descs


def _softmax_bw_rows(x: Tensor, oq_i: Tensor) -> int:
    L = x.shape[-1]
    if oq_i.numel() == 0:
        return 1
    _need(oq_i.numel() % L == 0, 'the output quantizer table must be [bw_rows, L]')
    return oq_i.numel() // L


@torch.library.custom_op('hgq::qsoftmax_fwd', mutates_args=())
def qsoftmax_fwd(x: Tensor, ks: Sequence[Tensor], is_: Sequence[Tensor], fbs: Sequence[Tensor], modes: Sequence[int],
                 input_scaler: float, eps: float, track_mask: int) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    _check_f32('x', x)
    _need(x.dim() >= 1 and 1 <= x.shape[-1] <= 256, 'softmax rows of 1..256 elements are supported')
    L = x.shape[-1]
    rows = x.numel() // L
    descs = _qdescs(ks, is_, fbs, modes)
    bw_rows = _softmax_bw_rows(x, is_[4])
    _need(rows % bw_rows == 0, 'rows must be a multiple of the output quantizer table rows')
    y = torch.empty_like(x)
    i32 = dict(dtype=torch.int32, device=x.device)
    a1 = torch.empty(1 if track_mask & 1 else 0, **i32)
    a3 = torch.empty(1 if track_mask & 2 else 0, **i32)
    ao = torch.empty(bw_rows * L if track_mask & 4 else 0, **i32)
    rc = _lib.load().hgq_qsoftmax_fwd(_ptr(x), _ptr(y), rows, L, bw_rows, input_scaler, eps,
                                      *[ctypes.addressof(d) for d in descs], _ptr(a1), _ptr(a3), _ptr(ao), _stream())
    _lib.check(rc, 'hgq_qsoftmax_fwd')
    return y, a1, a3, ao


@qsoftmax_fwd.register_fake
def _(x, ks, is_, fbs, modes, input_scaler, eps, track_mask):
    L = x.shape[-1]
    n_o = is_[4].numel() if track_mask & 4 else 0
    return (torch.empty_like(x), x.new_empty(1 if track_mask & 1 else 0, dtype=torch.int32),
            x.new_empty(1 if track_mask & 2 else 0, dtype=torch.int32), x.new_empty(n_o, dtype=torch.int32))


@torch.library.custom_op('hgq::qsoftmax_bwd', mutates_args=())
def qsoftmax_bwd(dy: Tensor, x: Tensor, ks: Sequence[Tensor], is_: Sequence[Tensor], fbs: Sequence[Tensor],
                 modes: Sequence[int], input_scaler: float, eps: float) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    _check_f32('dy', dy), _check_f32('x', x)
    _need(dy.shape == x.shape, 'dy and x differ in shape')
    L = x.shape[-1]
    rows = x.numel() // L
    descs = _qdescs(ks, is_, fbs, modes)
    has_oq = is_[4].numel() > 0
    bw_rows = _softmax_bw_rows(x, is_[4])
    lib = _lib.load()
    dx = torch.empty_like(x)
    f32 = dict(dtype=torch.float32, device=x.device)
    g_shared = torch.empty(8, **f32)
    g_oi = torch.empty(bw_rows * L if has_oq else 0, **f32)
    g_of = torch.empty(bw_rows * L if has_oq else 0, **f32)
    n_ws = lib.hgq_qsoftmax_bwd_workspace(rows, L, bw_rows, int(has_oq))
    _need(n_ws >= 0, 'hgq_qsoftmax_bwd_workspace rejected the shape')
    ws = torch.empty(max(int(n_ws), 1), **f32)
    rc = lib.hgq_qsoftmax_bwd(_ptr(dy), _ptr(x), _ptr(dx), rows, L, bw_rows, input_scaler, eps,
                              *[ctypes.addressof(d) for d in descs], _ptr(g_shared), _ptr(g_oi), _ptr(g_of), _ptr(ws), _stream())
    _lib.check(rc, 'hgq_qsoftmax_bwd')
    return dx, g_shared, g_oi, g_of


@qsoftmax_bwd.register_fake
def _(dy, x, ks, is_, fbs, modes, input_scaler, eps):
    n_o = is_[4].numel()
    return torch.empty_like(x), x.new_empty(8), x.new_empty(n_o), x.new_empty(n_o)


def _qattn_dims(q: Tensor, k: Tensor, v: Tensor):
    _check_f32('query', q), _check_f32('key', k), _check_f32('value', v)
    _need(q.dim() == 4 and k.dim() == 4 and v.shape == k.shape and q.shape[0] == k.shape[0] and q.shape[2:] == k.shape[2:],
          'query [B, T, N, H] and key / value [B, S, N, H] are expected')
    B, T, N, H = q.shape
    return B, T, k.shape[1], N, H


def _attn_bw_rows(S: int, oq_i: Tensor) -> int:
    if oq_i.numel() == 0:
        return 1
    _need(oq_i.numel() % S == 0, 'the output quantizer table must be [bw_rows, S]')
    return oq_i.numel() // S


def qattention_supported(q: Tensor, k: Tensor, v: Tensor, oq_entries: int, oq_saturates: bool) -> bool:
    """Whether ``qattention`` takes these operands (else compose attn_scores, qsoftmax, attn_combine)."""
    if not (q.is_cuda and q.dtype == torch.float32 and q.dim() == 4 and k.dim() == 4 and v.shape == k.shape) or oq_saturates:
        return False
    B, T, N, H = q.shape
    S = k.shape[1]
    if k.shape[0] != B or tuple(k.shape[2:]) != (N, H) or (oq_entries and oq_entries % S):
        return False
    return _lib.load().hgq_qattention_bwd_workspace(B, T, S, N, H, max(oq_entries // S, 1), int(oq_entries > 0)) >= 0


def _check_attn_mask(mask: Tensor, B: int, T: int, S: int):
    """An attention mask for the fused kernel: empty (none), or uint8 ``[1 or B, T, S]`` with 0 = masked out."""
    if mask.numel() == 0:
        return
    _need(mask.is_cuda and mask.dtype == torch.uint8 and mask.is_contiguous(), 'the attention mask must be a contiguous uint8 GPU tensor')
    _need(mask.dim() == 3 and mask.shape[0] in (1, B) and tuple(mask.shape[1:]) == (T, S),
          f'the attention mask must have shape [1 or {B}, {T}, {S}], got {tuple(mask.shape)}')


@torch.library.custom_op('hgq::qattention_fwd', mutates_args=())
def qattention_fwd(q: Tensor, k: Tensor, v: Tensor, ks: Sequence[Tensor], is_: Sequence[Tensor], fbs: Sequence[Tensor],
                   modes: Sequence[int], input_scaler: float, eps: float, track_mask: int, mask: Tensor,
                   causal: bool) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    B, T, S, N, H = _qattn_dims(q, k, v)
    _check_attn_mask(mask, B, T, S)
    descs = _qdescs(ks, is_, fbs, modes)
    bw_rows = _attn_bw_rows(S, is_[4])
    out = torch.empty_like(q)
    i32 = dict(dtype=torch.int32, device=q.device)
    a1 = torch.empty(1 if track_mask & 1 else 0, **i32)
    a3 = torch.empty(1 if track_mask & 2 else 0, **i32)
    ao = torch.empty(bw_rows * S if track_mask & 4 else 0, **i32)
    lib = _lib.load()
    n_ws = lib.hgq_qattention_fwd_workspace(B, T, S, N, H, bw_rows, int(bool(track_mask & 4)))
    _need(n_ws >= 0, 'hgq_qattention_fwd_workspace rejected the shape')
    ws = torch.empty(int(n_ws), **i32)
    rc = lib.hgq_qattention_fwd(_ptr(q), _ptr(k), _ptr(v), _ptr(out), B, T, S, N, H, bw_rows, input_scaler, eps,
                                *[ctypes.addressof(d) for d in descs], _ptr(a1), _ptr(a3), _ptr(ao), _ptr(ws), _ptr(mask),
                                mask.shape[0] if mask.numel() else 1, int(causal), _stream())
    _lib.check(rc, 'hgq_qattention_fwd')
    return out, a1, a3, ao


@qattention_fwd.register_fake
def _(q, k, v, ks, is_, fbs, modes, input_scaler, eps, track_mask, mask, causal):
    n_o = is_[4].numel() if track_mask & 4 else 0
    return (torch.empty_like(q), q.new_empty(1 if track_mask & 1 else 0, dtype=torch.int32),
            q.new_empty(1 if track_mask & 2 else 0, dtype=torch.int32), q.new_empty(n_o, dtype=torch.int32))


@torch.library.custom_op('hgq::qattention_bwd', mutates_args=())
def qattention_bwd(dout: Tensor, q: Tensor, k: Tensor, v: Tensor, ks: Sequence[Tensor], is_: Sequence[Tensor],
                   fbs: Sequence[Tensor], modes: Sequence[int], input_scaler: float, eps: float, mask: Tensor,
                   causal: bool) -> tuple[Tensor, Tensor, Tensor, Tensor, Tensor, Tensor]:
    B, T, S, N, H = _qattn_dims(q, k, v)
    _check_attn_mask(mask, B, T, S)
    _check_f32('dout', dout)
    _need(dout.shape == q.shape, 'dout and query differ in shape')
    descs = _qdescs(ks, is_, fbs, modes)
    has_oq = is_[4].numel() > 0
    bw_rows = _attn_bw_rows(S, is_[4])
    lib = _lib.load()
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    f32 = dict(dtype=torch.float32, device=q.device)
    g_shared = torch.empty(8, **f32)
    g_oi = torch.empty(bw_rows * S if has_oq else 0, **f32)
    g_of = torch.empty(bw_rows * S if has_oq else 0, **f32)
    n_ws = lib.hgq_qattention_bwd_workspace(B, T, S, N, H, bw_rows, int(has_oq))
    _need(n_ws >= 0, 'hgq_qattention_bwd_workspace rejected the shape')
    ws = torch.empty(max(int(n_ws), 1), **f32)
    rc = lib.hgq_qattention_bwd(_ptr(dout), _ptr(q), _ptr(k), _ptr(v), _ptr(dq), _ptr(dk), _ptr(dv), B, T, S, N, H, bw_rows,
                                input_scaler, eps, *[ctypes.addressof(d) for d in descs], _ptr(g_shared), _ptr(g_oi), _ptr(g_of),
                                _ptr(ws), _ptr(mask), mask.shape[0] if mask.numel() else 1, int(causal), _stream())
    _lib.check(rc, 'hgq_qattention_bwd')
    return dq, dk, dv, g_shared, g_oi, g_of


@qattention_bwd.register_fake
def _(dout, q, k, v, ks, is_, fbs, modes, input_scaler, eps, mask, causal):
    n_o = is_[4].numel()
    return torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), q.new_empty(8), q.new_empty(n_o), q.new_empty(n_o)


def _geom(g: Sequence[int]):
    _need(len(g) == 14, 'a convolution geometry has 14 entries (B, H, W, C, kh, kw, sy, sx, py, px, dly, dlx, OH, OW)')
    return _lib.ConvGeom(*[int(v) for v in g])


@torch.library.custom_op('hgq::conv2d_fwd', mutates_args=())
def conv2d_fwd(xq: Tensor, qw: Tensor, qb: Tensor, geom: Sequence[int], act: int) -> Tensor:
    _check_f32('xq', xq), _check_f32('qw', qw)
    g = _geom(geom)
    F = qw.shape[-1]
    _need(xq.numel() == g.B * g.H * g.W * g.C, f'input has {xq.numel()} elements, geometry says {g.B}x{g.H}x{g.W}x{g.C}')
    _need(qw.numel() == g.kh * g.kw * g.C * F, 'kernel must be [kh, kw, C, F]')
    if qb.numel():
        _check_f32('qb', qb)
        _need(qb.numel() == F, 'bias size mismatch')
    y = torch.empty((g.B, g.OH, g.OW, F), dtype=torch.float32, device=xq.device)
    lib = _lib.load()
    n_ws = lib.hgq_conv2d_fwd_workspace(ctypes.addressof(g), F)
    _need(n_ws >= 0, 'hgq_conv2d_fwd_workspace rejected the geometry')
    ws = torch.empty(int(n_ws), dtype=torch.float32, device=xq.device)
    rc = lib.hgq_conv2d_fwd(_ptr(xq), _ptr(qw), _ptr(qb), _ptr(y), _ptr(ws), ctypes.addressof(g), F, act, _stream())
    _lib.check(rc, 'hgq_conv2d_fwd')
    return y


@conv2d_fwd.register_fake
def _(xq, qw, qb, geom, act):
    return xq.new_empty((geom[0], geom[12], geom[13], qw.shape[-1]))


@torch.library.custom_op('hgq::conv2d_bwd', mutates_args=())
def conv2d_bwd(dy: Tensor, y: Tensor, xq: Tensor, qw: Tensor, geom: Sequence[int], act: int, need_dx: bool, has_bias: bool) -> tuple[Tensor, Tensor, Tensor]:
    _check_f32('dy', dy), _check_f32('y', y), _check_f32('xq', xq), _check_f32('qw', qw)
    g = _geom(geom)
    F = qw.shape[-1]
    _need(dy.numel() == g.B * g.OH * g.OW * F and y.numel() == dy.numel(), 'dy / y must be [B, OH, OW, F]')
    lib = _lib.load()
    f32 = dict(dtype=torch.float32, device=xq.device)
    dx = torch.empty(xq.shape if need_dx else (0,), **f32)
    dqw = torch.empty_like(qw)
    dqb = torch.empty(F if has_bias else 0, **f32)
    n_ws = lib.hgq_conv2d_bwd_workspace(ctypes.addressof(g), F)
    _need(n_ws >= 0, 'hgq_conv2d_bwd_workspace rejected the geometry')
    ws = torch.empty(max(int(n_ws), 1), **f32)
    rc = lib.hgq_conv2d_bwd(_ptr(dy), _ptr(y), _ptr(xq), _ptr(qw), _ptr(dx), _ptr(dqw), _ptr(dqb), _ptr(ws),
                            ctypes.addressof(g), F, act, _stream())
    _lib.check(rc, 'hgq_conv2d_bwd')
    return dx, dqw, dqb


@conv2d_bwd.register_fake
def _(dy, y, xq, qw, geom, act, need_dx, has_bias):
    return (xq.new_empty(xq.shape if need_dx else (0,)), torch.empty_like(qw), xq.new_empty(qw.shape[-1] if has_bias else 0))


@torch.library.custom_op('hgq::conv2d_bwd_slices', mutates_args=())
def conv2d_bwd_slices(dy: Tensor, y: Tensor, xq: Tensor, qw: Tensor, geom: Sequence[int], act: int, need_dx: bool) -> tuple[Tensor, Tensor]:
    """The convolution backward without the sum over its slices: ``(dx, slices [n, kh kw C F + F])``."""
    _check_f32('dy', dy), _check_f32('y', y), _check_f32('xq', xq), _check_f32('qw', qw)
    g = _geom(geom)
    F = qw.shape[-1]
    _need(dy.numel() == g.B * g.OH * g.OW * F and y.numel() == dy.numel(), 'dy / y must be [B, OH, OW, F]')
    lib = _lib.load()
    dx = torch.empty(xq.shape if need_dx else (0,), dtype=torch.float32, device=xq.device)
    n = lib.hgq_conv2d_bwd_slice_count(ctypes.addressof(g), F)
    _need(n >= 1, 'hgq_conv2d_bwd_slice_count rejected the geometry')
    ws = torch.empty((int(n), qw.numel() + F), dtype=torch.float32, device=xq.device)
    rc = lib.hgq_conv2d_bwd_slices(_ptr(dy), _ptr(y), _ptr(xq), _ptr(qw), _ptr(dx) if need_dx else None, _ptr(ws), ctypes.addressof(g), F,
                                   act, _stream())
    _lib.check(rc, 'hgq_conv2d_bwd_slices')
    return dx, ws


@conv2d_bwd_slices.register_fake
def _(dy, y, xq, qw, geom, act, need_dx):
    return xq.new_empty(xq.shape if need_dx else (0,)), xq.new_empty((1, qw.numel() + qw.shape[-1]))


@torch.library.custom_op('hgq::conv2d_maxpool_fwd', mutates_args=())
def conv2d_maxpool_fwd(xq: Tensor, qw: Tensor, qb: Tensor, geom: Sequence[int], act: int) -> tuple[Tensor, Tensor]:
    """``(y, maxpool2x2(y))`` with ``y = act(conv2d(xq, qw) + qb)`` in one launch (``qb`` empty: no bias)."""
    _check_f32('xq', xq), _check_f32('qw', qw), _check_f32('qb', qb)
    g = _geom(geom)
    F = qw.shape[-1]
    _need(xq.numel() == g.B * g.H * g.W * g.C and tuple(qw.shape) == (g.kh, g.kw, g.C, F), 'xq / qw do not match the geometry')
    _need(qb.numel() in (0, F), 'qb must hold one entry per filter')
    y = torch.empty((g.B, g.OH, g.OW, F), dtype=torch.float32, device=xq.device)
    yp = torch.empty((g.B, g.OH // 2, g.OW // 2, F), dtype=torch.float32, device=xq.device)
    rc = _lib.load().hgq_conv2d_maxpool_fwd(_ptr(xq), _ptr(qw), _ptr(qb) if qb.numel() else None, _ptr(y), _ptr(yp), ctypes.addressof(g),
                                            F, act, _stream())
    _lib.check(rc, 'hgq_conv2d_maxpool_fwd')
    return y, yp


@conv2d_maxpool_fwd.register_fake
def _(xq, qw, qb, geom, act):
    F = qw.shape[-1]
    return xq.new_empty((geom[0], geom[12], geom[13], F)), xq.new_empty((geom[0], geom[12] // 2, geom[13] // 2, F))


@torch.library.custom_op('hgq::conv2d_maxpool_bwd', mutates_args=())
def conv2d_maxpool_bwd(dyp: Tensor, y: Tensor, xq: Tensor, qw: Tensor, geom: Sequence[int], act: int, need_dx: bool,
                       reduce: bool) -> tuple[Tensor, Tensor]:
    """Backward of a convolution behind a 2 x 2 / stride 2 / unpadded maximum pooling from the pooled gradient ``dyp``:
    ``(dx, slices [n, kh kw C F + F])``, or with ``reduce`` ``(dx, [kh kw C F + F])`` (kernel gradient, then bias gradient)."""
    _check_f32('dyp', dyp), _check_f32('y', y), _check_f32('xq', xq), _check_f32('qw', qw)
    g = _geom(geom)
    F = qw.shape[-1]
    _need(y.numel() == g.B * g.OH * g.OW * F, 'y must be [B, OH, OW, F]')
    _need(dyp.numel() == g.B * (g.OH // 2) * (g.OW // 2) * F, 'dyp must be [B, OH // 2, OW // 2, F]')
    lib = _lib.load()
    dx = torch.empty(xq.shape if need_dx else (0,), dtype=torch.float32, device=xq.device)
    n = lib.hgq_conv2d_bwd_slice_count(ctypes.addressof(g), F)
    _need(n >= 1, 'hgq_conv2d_bwd_slice_count rejected the geometry')
    ws = torch.empty((int(n), qw.numel() + F), dtype=torch.float32, device=xq.device)
    out = torch.empty(qw.numel() + F, dtype=torch.float32, device=xq.device) if reduce else ws
    rc = lib.hgq_conv2d_maxpool_bwd(_ptr(dyp), _ptr(y), _ptr(xq), _ptr(qw), _ptr(dx) if need_dx else None, _ptr(out),
                                    out.data_ptr() + 4 * qw.numel() if reduce else None, _ptr(ws), ctypes.addressof(g), F, act,
                                    int(reduce), _stream())
    _lib.check(rc, 'hgq_conv2d_maxpool_bwd')
    return dx, out


@conv2d_maxpool_bwd.register_fake
def _(dyp, y, xq, qw, geom, act, need_dx, reduce):
    n = qw.numel() + qw.shape[-1]
    return xq.new_empty(xq.shape if need_dx else (0,)), xq.new_empty((n,) if reduce else (1, n))


@torch.library.custom_op('hgq::conv2d_maxpool_fwd_coded', mutates_args=())
def conv2d_maxpool_fwd_coded(xq: Tensor, qw: Tensor, qb: Tensor, geom: Sequence[int], act: int) -> tuple[Tensor, Tensor]:
    """``(code, maxpool2x2(act(conv2d(xq, qw) + qb)))`` in one launch; the unpooled tensor is never written.  ``code`` (uint8,
    the pooled shape): bits 0-1 the row-major place of each window's first maximum, bit 2 whether it is positive."""
    _check_f32('xq', xq), _check_f32('qw', qw), _check_f32('qb', qb)
    g = _geom(geom)
    F = qw.shape[-1]
    _need(xq.numel() == g.B * g.H * g.W * g.C and tuple(qw.shape) == (g.kh, g.kw, g.C, F), 'xq / qw do not match the geometry')
    _need(qb.numel() in (0, F), 'qb must hold one entry per filter')
    code = torch.empty((g.B, g.OH // 2, g.OW // 2, F), dtype=torch.uint8, device=xq.device)
    yp = torch.empty((g.B, g.OH // 2, g.OW // 2, F), dtype=torch.float32, device=xq.device)
    rc = _lib.load().hgq_conv2d_maxpool_fwd_coded(_ptr(xq), _ptr(qw), _ptr(qb) if qb.numel() else None, _ptr(yp), _ptr(code),
                                                  ctypes.addressof(g), F, act, _stream())
    _lib.check(rc, 'hgq_conv2d_maxpool_fwd_coded')
    return code, yp


@conv2d_maxpool_fwd_coded.register_fake
def _(xq, qw, qb, geom, act):
    F = qw.shape[-1]
    shape = (geom[0], geom[12] // 2, geom[13] // 2, F)
    return xq.new_empty(shape, dtype=torch.uint8), xq.new_empty(shape)


@torch.library.custom_op('hgq::conv2d_maxpool_bwd_coded', mutates_args=())
def conv2d_maxpool_bwd_coded(dyp: Tensor, code: Tensor, xq: Tensor, qw: Tensor, geom: Sequence[int], act: int, need_dx: bool,
                             reduce: bool) -> tuple[Tensor, Tensor]:
    """``conv2d_maxpool_bwd`` from the forward pass's window codes instead of its unpooled output."""
    _check_f32('dyp', dyp), _check_f32('xq', xq), _check_f32('qw', qw)
    g = _geom(geom)
    F = qw.shape[-1]
    n_p = g.B * (g.OH // 2) * (g.OW // 2) * F
    _need(code.dtype == torch.uint8 and code.is_contiguous() and code.numel() == n_p, 'code must be uint8 [B, OH // 2, OW // 2, F]')
    _need(dyp.numel() == n_p, 'dyp must be [B, OH // 2, OW // 2, F]')
    lib = _lib.load()
    dx = torch.empty(xq.shape if need_dx else (0,), dtype=torch.float32, device=xq.device)
    n = lib.hgq_conv2d_bwd_slice_count(ctypes.addressof(g), F)
    _need(n >= 1, 'hgq_conv2d_bwd_slice_count rejected the geometry')
    ws = torch.empty((int(n), qw.numel() + F), dtype=torch.float32, device=xq.device)
    out = torch.empty(qw.numel() + F, dtype=torch.float32, device=xq.device) if reduce else ws
    rc = lib.hgq_conv2d_maxpool_bwd_coded(_ptr(dyp), _ptr(code), _ptr(xq), _ptr(qw), _ptr(dx) if need_dx else None, _ptr(out),
                                          out.data_ptr() + 4 * qw.numel() if reduce else None, _ptr(ws), ctypes.addressof(g), F, act,
                                          int(reduce), _stream())
    _lib.check(rc, 'hgq_conv2d_maxpool_bwd_coded')
    return dx, out


@conv2d_maxpool_bwd_coded.register_fake
def _(dyp, code, xq, qw, geom, act, need_dx, reduce):
    n = qw.numel() + qw.shape[-1]
    return xq.new_empty(xq.shape if need_dx else (0,)), xq.new_empty((n,) if reduce else (1, n))


def conv2d_maxpool_supported(geom, F: int) -> bool:
    g = _geom(geom)
    return bool(_lib.load().hgq_conv2d_maxpool_bwd_supported(ctypes.addressof(g), int(F)))


@torch.library.custom_op('hgq::col_moments_fwd', mutates_args=())
def col_moments_fwd(x: Tensor) -> tuple[Tensor, Tensor]:
    _check_f32('x', x)
    _need(x.dim() == 2 and x.shape[0] >= 1, 'x must be [rows >= 1, N]')
    rows, N = x.shape
    lib = _lib.load()
    mean = torch.empty(N, dtype=torch.float32, device=x.device)
    meansq = torch.empty(N, dtype=torch.float32, device=x.device)
    ws = torch.empty(int(lib.hgq_col_moments_workspace(rows, N)), dtype=torch.float32, device=x.device)
    rc = lib.hgq_col_moments_fwd(_ptr(x), rows, N, _ptr(mean), _ptr(meansq), _ptr(ws), _stream())
    _lib.check(rc, 'hgq_col_moments_fwd')
    return mean, meansq


@col_moments_fwd.register_fake
def _(x):
    return x.new_empty(x.shape[1]), x.new_empty(x.shape[1])


@torch.library.custom_op('hgq::col_moments_bwd', mutates_args=())
def col_moments_bwd(x: Tensor, dmean: Tensor, dmeansq: Tensor) -> Tensor:
    _check_f32('x', x), _check_f32('dmean', dmean), _check_f32('dmeansq', dmeansq)
    rows, N = x.shape
    _need(dmean.numel() == N and dmeansq.numel() == N, 'gradient size mismatch')
    dx = torch.empty_like(x)
    rc = _lib.load().hgq_col_moments_bwd(_ptr(x), _ptr(dmean), _ptr(dmeansq), rows, N, _ptr(dx), _stream())
    _lib.check(rc, 'hgq_col_moments_bwd')
    return dx


@col_moments_bwd.register_fake
def _(x, dmean, dmeansq):
    return torch.empty_like(x)


ATTN_MAX = 64  # the attention contraction kernels cover sequence lengths and head sizes up to 64


def _attn_dims(a: Tensor, b: Tensor):
    """a [B, T, N, H], b [B, S, N, H] -> (B, T, S, N, H)"""
    _need(a.dim() == 4 and b.dim() == 4 and a.shape[0] == b.shape[0] and a.shape[2:] == b.shape[2:], 'operands must be [B, seq, N, H]')
    return a.shape[0], a.shape[1], b.shape[1], a.shape[2], a.shape[3]


@torch.library.custom_op('hgq::attn_scores_fwd', mutates_args=())
def attn_scores_fwd(query: Tensor, key: Tensor) -> Tensor:
    _check_f32('query', query), _check_f32('key', key)
    B, T, S, N, H = _attn_dims(query, key)
    scores = torch.empty((B, N, T, S), dtype=torch.float32, device=query.device)
    rc = _lib.load().hgq_attn_scores_fwd(_ptr(query), _ptr(key), _ptr(scores), B, T, S, N, H, _stream())
    _lib.check(rc, 'hgq_attn_scores_fwd')
    return scores


@attn_scores_fwd.register_fake
def _(query, key):
    return query.new_empty((query.shape[0], query.shape[2], query.shape[1], key.shape[1]))


@torch.library.custom_op('hgq::attn_scores_bwd', mutates_args=())
def attn_scores_bwd(dscores: Tensor, query: Tensor, key: Tensor) -> tuple[Tensor, Tensor]:
    _check_f32('dscores', dscores), _check_f32('query', query), _check_f32('key', key)
    B, T, S, N, H = _attn_dims(query, key)
    _need(tuple(dscores.shape) == (B, N, T, S), 'dscores must be [B, N, T, S]')
    dq, dk = torch.empty_like(query), torch.empty_like(key)
    rc = _lib.load().hgq_attn_scores_bwd(_ptr(dscores), _ptr(query), _ptr(key), _ptr(dq), _ptr(dk), B, T, S, N, H, _stream())
    _lib.check(rc, 'hgq_attn_scores_bwd')
    return dq, dk


@attn_scores_bwd.register_fake
def _(dscores, query, key):
    return torch.empty_like(query), torch.empty_like(key)


@torch.library.custom_op('hgq::attn_combine_fwd', mutates_args=())
def attn_combine_fwd(probs: Tensor, value: Tensor) -> Tensor:
    _check_f32('probs', probs), _check_f32('value', value)
    _need(probs.dim() == 4 and value.dim() == 4, 'probs [B, N, T, S], value [B, S, N, H]')
    B, N, T, S = probs.shape
    _need(value.shape[0] == B and value.shape[1] == S and value.shape[2] == N, 'value must be [B, S, N, H]')
    H = value.shape[3]
    out = torch.empty((B, T, N, H), dtype=torch.float32, device=probs.device)
    rc = _lib.load().hgq_attn_combine_fwd(_ptr(probs), _ptr(value), _ptr(out), B, T, S, N, H, _stream())
    _lib.check(rc, 'hgq_attn_combine_fwd')
    return out


@attn_combine_fwd.register_fake
def _(probs, value):
    return probs.new_empty((probs.shape[0], probs.shape[2], probs.shape[1], value.shape[3]))


@torch.library.custom_op('hgq::attn_combine_bwd', mutates_args=())
def attn_combine_bwd(dout: Tensor, probs: Tensor, value: Tensor) -> tuple[Tensor, Tensor]:
    _check_f32('dout', dout), _check_f32('probs', probs), _check_f32('value', value)
    B, N, T, S = probs.shape
    H = value.shape[3]
    _need(tuple(dout.shape) == (B, T, N, H), 'dout must be [B, T, N, H]')
    dp, dv = torch.empty_like(probs), torch.empty_like(value)
    rc = _lib.load().hgq_attn_combine_bwd(_ptr(dout), _ptr(probs), _ptr(value), _ptr(dp), _ptr(dv), B, T, S, N, H, _stream())
    _lib.check(rc, 'hgq_attn_combine_bwd')
    return dp, dv


@attn_combine_bwd.register_fake
def _(dout, probs, value):
    return torch.empty_like(probs), torch.empty_like(value)


@torch.library.custom_op('hgq::pool2d_fwd', mutates_args=())
def pool2d_fwd(x: Tensor, geom: Sequence[int], is_max: bool) -> Tensor:
    _check_f32('x', x)
    _need(len(geom) == 12 and x.numel() == geom[0] * geom[1] * geom[2] * geom[3], 'x must be [B, H, W, C] as in the geometry')
    y = torch.empty((geom[0], geom[10], geom[11], geom[3]), dtype=torch.float32, device=x.device)
    g = (ctypes.c_int * 12)(*[int(v) for v in geom])
    rc = _lib.load().hgq_pool2d_fwd(_ptr(x), _ptr(y), g, int(is_max), _stream())
    _lib.check(rc, 'hgq_pool2d_fwd')
    return y


@pool2d_fwd.register_fake
def _(x, geom, is_max):
    return x.new_empty((geom[0], geom[10], geom[11], geom[3]))


@torch.library.custom_op('hgq::pool2d_bwd', mutates_args=())
def pool2d_bwd(dy: Tensor, x: Tensor, geom: Sequence[int], is_max: bool) -> Tensor:
    _check_f32('dy', dy), _check_f32('x', x)
    _need(dy.numel() == geom[0] * geom[10] * geom[11] * geom[3], 'dy must be [B, OH, OW, C] as in the geometry')
    dx = torch.empty_like(x)
    g = (ctypes.c_int * 12)(*[int(v) for v in geom])
    rc = _lib.load().hgq_pool2d_bwd(_ptr(dy), _ptr(x), _ptr(dx), g, int(is_max), _stream())
    _lib.check(rc, 'hgq_pool2d_bwd')
    return dx


@pool2d_bwd.register_fake
def _(dy, x, geom, is_max):
    return torch.empty_like(x)


@torch.library.custom_op('hgq::mean_mid_fwd', mutates_args=())
def mean_mid_fwd(x: Tensor) -> Tensor:
    _check_f32('x', x)
    _need(x.dim() == 3, 'x must be [B, P, N]')
    B, P, N = x.shape
    y = torch.empty((B, N), dtype=torch.float32, device=x.device)
    _lib.check(_lib.load().hgq_mean_mid_fwd(_ptr(x), _ptr(y), B, P, N, _stream()), 'hgq_mean_mid_fwd')
    return y


@mean_mid_fwd.register_fake
def _(x):
    return x.new_empty((x.shape[0], x.shape[2]))


@torch.library.custom_op('hgq::mean_mid_bwd', mutates_args=())
def mean_mid_bwd(dy: Tensor, P: int) -> Tensor:
    _check_f32('dy', dy)
    B, N = dy.shape
    dx = torch.empty((B, P, N), dtype=torch.float32, device=dy.device)
    _lib.check(_lib.load().hgq_mean_mid_bwd(_ptr(dy), _ptr(dx), B, P, N, _stream()), 'hgq_mean_mid_bwd')
    return dx


@mean_mid_bwd.register_fake
def _(dy, P):
    return dy.new_empty((dy.shape[0], P, dy.shape[1]))


class _MeanMid(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        ctx.P = x.shape[1]
        return mean_mid_fwd(x)

    @staticmethod
    def backward(ctx, g):
        return mean_mid_bwd(g.contiguous(), ctx.P)


def mean_mid(x: Tensor) -> Tensor:
    """``x.mean(1)`` of a ``[B, P, N]`` GPU tensor (one pass each way, rows added in a fixed order)."""
    return _MeanMid.apply(x.contiguous())


def conv2d_ebops_supported(in_shape, kernel_shape) -> bool:
    """Whether hgq_conv2d_ebops covers bit-width tensors [1, H, W, C] x [kh, kw, C, F] (its LDS tables bound the sizes)."""
    _, H, W, C = in_shape
    kh, kw, F = kernel_shape[0], kernel_shape[1], kernel_shape[3]
    return (kh * kw * C <= 4096 and kh * W * C <= 8192 and H * kh <= 2048 and W * kw <= 2048 and kh * kw * C * F < 2**21
            and H * W * C < 2**21)


@torch.library.custom_op('hgq::conv2d_ebops', mutates_args=())
def conv2d_ebops_op(bits_in: Tensor, bits_ker: Tensor, geom: Sequence[int]) -> tuple[Tensor, Tensor, Tensor]:
    _check_f32('bits_in', bits_in), _check_f32('bits_ker', bits_ker)
    g = _geom(geom)
    F = bits_ker.shape[-1]
    _need(bits_in.numel() == g.H * g.W * g.C and bits_ker.numel() == g.kh * g.kw * g.C * F, 'bit-width tensors do not match the geometry')
    total = torch.empty((), dtype=torch.float32, device=bits_in.device)
    g_in, g_ker = torch.empty_like(bits_in), torch.empty_like(bits_ker)
    rc = _lib.load().hgq_conv2d_ebops(_ptr(bits_in), _ptr(bits_ker), ctypes.addressof(g), F, _ptr(total), _ptr(g_in), _ptr(g_ker), _stream())
    _lib.check(rc, 'hgq_conv2d_ebops')
    return total, g_in, g_ker


@conv2d_ebops_op.register_fake
def _(bits_in, bits_ker, geom):
    return bits_in.new_empty(()), torch.empty_like(bits_in), torch.empty_like(bits_ker)


@torch.library.custom_op('hgq::mse_fwd', mutates_args=())
def mse_fwd_op(pred: Tensor, target: Tensor) -> Tensor:
    _check_f32('pred', pred)
    if target.numel():
        _check_f32('target', target)
        _need(target.numel() == pred.numel(), 'target size mismatch')
    lib = _lib.load()
    loss = torch.empty((), dtype=torch.float32, device=pred.device)
    ws = torch.empty(lib.hgq_mse_workspace(), dtype=torch.float32, device=pred.device)
    _lib.check(lib.hgq_mse_fwd(_ptr(pred), _ptr(target), _ptr(loss), _ptr(ws), pred.numel(), _stream()), 'hgq_mse_fwd')
    return loss


@mse_fwd_op.register_fake
def _(pred, target):
    return pred.new_empty(())


@torch.library.custom_op('hgq::mse_fwd_bwd', mutates_args=())
def mse_fwd_bwd_op(pred: Tensor, target: Tensor) -> tuple[Tensor, Tensor]:
    """``(loss, dpred for a unit upstream gradient)`` in one pass over the operands."""
    _check_f32('pred', pred)
    if target.numel():
        _check_f32('target', target)
        _need(target.numel() == pred.numel(), 'target size mismatch')
    lib = _lib.load()
    loss = torch.empty((), dtype=torch.float32, device=pred.device)
    dpred = torch.empty_like(pred)
    ws = torch.empty(lib.hgq_mse_workspace(), dtype=torch.float32, device=pred.device)
    _lib.check(lib.hgq_mse_fwd_bwd(_ptr(pred), _ptr(target), _ptr(loss), _ptr(dpred), _ptr(ws), pred.numel(), _stream()), 'hgq_mse_fwd_bwd')
    return loss, dpred


@mse_fwd_bwd_op.register_fake
def _(pred, target):
    return pred.new_empty(()), torch.empty_like(pred)


def dense_moments_supported(x2d: Tensor, w2d: Tensor) -> bool:
    """Whether hgq_dense_moments_* covers this contraction (K, N <= 64, multiples of 4, aligned input)."""
    K, N = w2d.shape
    return x2d.is_cuda and x2d.shape[0] > 0 and K <= 64 and N <= 64 and K % 4 == 0 and N % 4 == 0 and x2d.data_ptr() % 16 == 0


@torch.library.custom_op('hgq::dense_moments_fwd', mutates_args=())
def dense_moments_fwd(x: Tensor, w: Tensor, f_in: Tensor, bw_rows: int, mode: int) -> tuple[Tensor, Tensor]:
    _check_f32('x', x), _check_f32('w', w)
    _need(x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[0], 'shape mismatch')
    rows, K = x.shape
    N = w.shape[1]
    if bw_rows:
        _check_f32('f_in', f_in)
        _need(f_in.numel() == bw_rows * K, 'f_in must be a [bw_rows, K] table')
    lib = _lib.load()
    mean, meansq = (torch.empty(N, dtype=torch.float32, device=x.device) for _ in range(2))
    ws = torch.empty(max(lib.hgq_qdense_moments_workspace(rows, K, N, bw_rows), 1), dtype=torch.float32, device=x.device)
    _lib.check(lib.hgq_qdense_moments_fwd(_ptr(x), _ptr(f_in), bw_rows, mode, _ptr(w), _ptr(mean), _ptr(meansq), _ptr(ws), rows, K, N,
                                          _stream()), 'hgq_qdense_moments_fwd')
    return mean, meansq


@dense_moments_fwd.register_fake
def _(x, w, f_in, bw_rows, mode):
    return x.new_empty(w.shape[1]), x.new_empty(w.shape[1])


@torch.library.custom_op('hgq::dense_moments_bwd', mutates_args=())
def dense_moments_bwd(x: Tensor, w: Tensor, f_in: Tensor, bw_rows: int, mode: int, dmean: Tensor,
                      dmeansq: Tensor, dx_add: Tensor) -> tuple[Tensor, Tensor, Tensor]:
    _check_f32('x', x), _check_f32('w', w), _check_f32('dmean', dmean), _check_f32('dmeansq', dmeansq)
    if dx_add.numel():
        _check_f32('dx_add', dx_add)
        _need(dx_add.shape == x.shape, 'dx_add must have the shape of x')
    rows, K = x.shape
    N = w.shape[1]
    lib = _lib.load()
    dx, dw = torch.empty_like(x), torch.empty_like(w)
    df = torch.empty(bw_rows * K, dtype=torch.float32, device=x.device)
    ws = torch.empty(max(lib.hgq_qdense_moments_workspace(rows, K, N, bw_rows), 1), dtype=torch.float32, device=x.device)
    _lib.check(lib.hgq_qdense_moments_bwd(_ptr(x), _ptr(f_in), bw_rows, mode, _ptr(w), _ptr(dmean), _ptr(dmeansq), _ptr(dx_add), _ptr(dx),
                                          _ptr(dw), _ptr(df), _ptr(ws), rows, K, N, _stream()), 'hgq_qdense_moments_bwd')
    return dx, dw, df


@dense_moments_bwd.register_fake
def _(x, w, f_in, bw_rows, mode, dmean, dmeansq, dx_add):
    return torch.empty_like(x), torch.empty_like(w), x.new_empty(bw_rows * x.shape[1])


@torch.library.custom_op('hgq::dense_moments_bwd_slices', mutates_args=())
def dense_moments_bwd_slices(x: Tensor, w: Tensor, f_in: Tensor, bw_rows: int, mode: int, dmean: Tensor, dmeansq: Tensor,
                             dx_add: Tensor) -> tuple[Tensor, Tensor]:
    """``dense_moments_bwd`` without the sum over its slices: ``(dx, slices [n, K*N + N + bw_rows*K])`` (the N section unused)."""
    _check_f32('x', x), _check_f32('w', w), _check_f32('dmean', dmean), _check_f32('dmeansq', dmeansq)
    if dx_add.numel():
        _check_f32('dx_add', dx_add)
        _need(dx_add.shape == x.shape, 'dx_add must have the shape of x')
    rows, K = x.shape
    N = w.shape[1]
    lib = _lib.load()
    dx = torch.empty_like(x)
    width = K * N + N + bw_rows * K
    ws = torch.empty((lib.hgq_qdense_bwd_workspace(rows, K, N, bw_rows) // width, width), dtype=torch.float32, device=x.device)
    _lib.check(lib.hgq_qdense_moments_bwd(_ptr(x), _ptr(f_in), bw_rows, mode, _ptr(w), _ptr(dmean), _ptr(dmeansq), _ptr(dx_add), _ptr(dx),
                                          None, None, _ptr(ws), rows, K, N, _stream()), 'hgq_qdense_moments_bwd')
    return dx, ws


@dense_moments_bwd_slices.register_fake
def _(x, w, f_in, bw_rows, mode, dmean, dmeansq, dx_add):
    K, N = w.shape
    return torch.empty_like(x), x.new_empty((1, K * N + N + bw_rows * K))


@torch.library.custom_op('hgq::bn_fold_fwd', mutates_args=('moving_mean', 'moving_var'))
def bn_fold_fwd(w: Tensor, bias: Tensor, gamma: Tensor, mean: Tensor, second: Tensor, is_meansq: bool, eps: float,
                moving_mean: Tensor, moving_var: Tensor, momentum: float) -> tuple[Tensor, Tensor]:
    for name, t in (('w', w), ('bias', bias), ('mean', mean), ('second', second)):
        _check_f32(name, t)
    K, N = w.shape
    _need(bias.numel() == N and mean.numel() == N and second.numel() == N and gamma.numel() in (0, N), 'per-column operands must have N entries')
    _need(moving_mean.numel() in (0, N) and moving_var.numel() in (0, N), 'moving statistics must have N entries')
    fw, fb = torch.empty_like(w), torch.empty_like(bias)
    rc = _lib.load().hgq_bn_fold_fwd(_ptr(w), _ptr(bias), _ptr(gamma), _ptr(mean), _ptr(second), int(is_meansq), eps, _ptr(fw), _ptr(fb),
                                     _ptr(moving_mean), _ptr(moving_var), momentum, 1.0 - momentum, K, N, _stream())
    _lib.check(rc, 'hgq_bn_fold_fwd')
    return fw, fb


@bn_fold_fwd.register_fake
def _(w, bias, gamma, mean, second, is_meansq, eps, moving_mean, moving_var, momentum):
    return torch.empty_like(w), torch.empty_like(bias)


@torch.library.custom_op('hgq::bn_fold_bwd', mutates_args=())
def bn_fold_bwd(w: Tensor, gamma: Tensor, mean: Tensor, second: Tensor, is_meansq: bool, eps: float, d_fw: Tensor,
                d_fb: Tensor) -> tuple[Tensor, Tensor, Tensor, Tensor, Tensor]:
    _check_f32('d_fw', d_fw), _check_f32('d_fb', d_fb)
    K, N = w.shape
    dw = torch.empty_like(w)
    dbias, dmean, dsecond = (torch.empty(N, dtype=torch.float32, device=w.device) for _ in range(3))
    dgamma = torch.empty(N if gamma.numel() else 0, dtype=torch.float32, device=w.device)
    rc = _lib.load().hgq_bn_fold_bwd(_ptr(w), _ptr(gamma), _ptr(mean), _ptr(second), int(is_meansq), eps, _ptr(d_fw), _ptr(d_fb), _ptr(dw),
                                     _ptr(dbias), _ptr(dgamma), _ptr(dmean), _ptr(dsecond), K, N, _stream())
    _lib.check(rc, 'hgq_bn_fold_bwd')
    return dw, dbias, dgamma, dmean, dsecond


@bn_fold_bwd.register_fake
def _(w, gamma, mean, second, is_meansq, eps, d_fw, d_fb):
    n = w.shape[1]
    return torch.empty_like(w), w.new_empty(n), w.new_empty(n if gamma.numel() else 0), w.new_empty(n), w.new_empty(n)


def _qdesc(k: Tensor, i: Tensor, fb: Tensor, mode: int):
    return _lib.QDesc(k.data_ptr(), i.data_ptr(), fb.data_ptr(), _kmode(mode, k))


@torch.library.custom_op('hgq::bn_fold_quant_fwd', mutates_args=('moving_mean', 'moving_var'))
def bn_fold_quant_fwd(w: Tensor, bias: Tensor, gamma: Tensor, mean: Tensor, second: Tensor, is_meansq: bool, eps: float,
                      moving_mean: Tensor, moving_var: Tensor, momentum: float, qk: Sequence[Tensor], qb: Sequence[Tensor],
                      modes: Sequence[int]) -> tuple[Tensor, Tensor]:
    """``bn_fold_fwd`` followed, in the same launch, by the kernel and bias quantizers ``qk`` / ``qb`` = ``(k, i, fb)``:
    returns the quantized folded kernel and bias."""
    for name, t in (('w', w), ('bias', bias), ('mean', mean), ('second', second)):
        _check_f32(name, t)
    K, N = w.shape
    _need(bias.numel() == N and mean.numel() == N and second.numel() == N and gamma.numel() in (0, N), 'per-column operands must have N entries')
    _need(moving_mean.numel() in (0, N) and moving_var.numel() in (0, N), 'moving statistics must have N entries')
    _need(all(t.numel() == K * N for t in qk) and all(t.numel() == N for t in qb), 'quantizer operands must match the kernel and the bias')
    dk, db = _qdesc(*qk, modes[0]), _qdesc(*qb, modes[1])
    qw, qbias = torch.empty_like(w), torch.empty_like(bias)
    rc = _lib.load().hgq_bn_fold_quant_fwd(_ptr(w), _ptr(bias), _ptr(gamma), _ptr(mean), _ptr(second), int(is_meansq), eps,
                                           ctypes.addressof(dk), ctypes.addressof(db), _ptr(qw), _ptr(qbias), _ptr(moving_mean),
                                           _ptr(moving_var), momentum, 1.0 - momentum, K, N, _stream())
    _lib.check(rc, 'hgq_bn_fold_quant_fwd')
    return qw, qbias


@bn_fold_quant_fwd.register_fake
def _(w, bias, gamma, mean, second, is_meansq, eps, moving_mean, moving_var, momentum, qk, qb, modes):
    return torch.empty_like(w), torch.empty_like(bias)


@torch.library.custom_op('hgq::bn_fold_quant_bwd', mutates_args=())
def bn_fold_quant_bwd(w: Tensor, bias: Tensor, gamma: Tensor, mean: Tensor, second: Tensor, is_meansq: bool, eps: float, d_qw: Tensor,
                      d_qb: Tensor, qk: Sequence[Tensor], qb: Sequence[Tensor], modes: Sequence[int]) -> list[Tensor]:
    """Backward of ``bn_fold_quant_fwd``: ``[dw, dbias, dgamma, dmean, dsecond, di_k, dfb_k, di_b, dfb_b]``."""
    _check_f32('d_qw', d_qw), _check_f32('d_qb', d_qb)
    K, N = w.shape
    dev = w.device
    dw, di_k, dfb_k = torch.empty_like(w), torch.empty_like(w), torch.empty_like(w)
    dbias, dmean, dsecond, di_b, dfb_b = (torch.empty(N, dtype=torch.float32, device=dev) for _ in range(5))
    dgamma = torch.empty(N if gamma.numel() else 0, dtype=torch.float32, device=dev)
    dk, db = _qdesc(*qk, modes[0]), _qdesc(*qb, modes[1])
    rc = _lib.load().hgq_bn_fold_quant_bwd(_ptr(w), _ptr(bias), _ptr(gamma), _ptr(mean), _ptr(second), int(is_meansq), eps,
                                           ctypes.addressof(dk), ctypes.addressof(db), _ptr(d_qw), _ptr(d_qb), _ptr(dw), _ptr(dbias),
                                           _ptr(dgamma), _ptr(dmean), _ptr(dsecond), _ptr(di_k), _ptr(dfb_k), _ptr(di_b), _ptr(dfb_b), K, N,
                                           _stream())
    _lib.check(rc, 'hgq_bn_fold_quant_bwd')
    return [dw, dbias, dgamma, dmean, dsecond, di_k, dfb_k, di_b, dfb_b]


@bn_fold_quant_bwd.register_fake
def _(w, bias, gamma, mean, second, is_meansq, eps, d_qw, d_qb, qk, qb, modes):
    n = w.shape[1]
    return ([torch.empty_like(w), w.new_empty(n), w.new_empty(n if gamma.numel() else 0), w.new_empty(n), w.new_empty(n),
             torch.empty_like(w), torch.empty_like(w), w.new_empty(n), w.new_empty(n)])


@torch.library.custom_op('hgq::qbits_fwd', mutates_args=())
def qbits_fwd(k: Tensor, i: Tensor, fb: Tensor, kbi: bool, add_mode: int) -> Tensor:
    _check_f32('fb', fb)
    n = fb.numel()
    if not kbi:
        _check_f32('i', i)
        _need(i.numel() == n, 'i / f size mismatch')
    if add_mode:
        _need(k.dtype == torch.uint8 and k.is_cuda and k.is_contiguous() and k.numel() == n, 'k must be a contiguous uint8 GPU tensor of the same size')
    out = torch.empty_like(fb)
    _lib.check(_lib.load().hgq_qbits_fwd(_ptr(k), _ptr(i), _ptr(fb), n, int(kbi), add_mode, _ptr(out), _stream()), 'hgq_qbits_fwd')
    return out


@qbits_fwd.register_fake
def _(k, i, fb, kbi, add_mode):
    return torch.empty_like(fb)


@torch.library.custom_op('hgq::qbits_bwd', mutates_args=())
def qbits_bwd(g: Tensor, i: Tensor, fb: Tensor, kbi: bool) -> tuple[Tensor, Tensor]:
    _check_f32('g', g)
    dfb = torch.empty_like(fb)
    di = torch.empty_like(fb) if not kbi else fb.new_empty(0)
    _lib.check(_lib.load().hgq_qbits_bwd(_ptr(g), _ptr(i), _ptr(fb), fb.numel(), int(kbi), _ptr(di), _ptr(dfb), _stream()), 'hgq_qbits_bwd')
    return di, dfb


@qbits_bwd.register_fake
def _(g, i, fb, kbi):
    return (torch.empty_like(fb) if not kbi else fb.new_empty(0)), torch.empty_like(fb)


@torch.library.custom_op('hgq::ebops_finish_fwd', mutates_args=('ebops_var',))
def ebops_finish_fwd(ebops: Tensor, factor: float, beta: Tensor, ebops_var: Tensor) -> Tensor:
    _check_f32('ebops', ebops), _check_f32('beta', beta)
    _need(ebops.numel() == 1 and beta.numel() == 1 and ebops_var.numel() == 1 and ebops_var.element_size() == 4, 'scalars expected')
    out = torch.empty((), dtype=torch.float32, device=ebops.device)
    _lib.check(_lib.load().hgq_ebops_finish_fwd(_ptr(ebops), factor, _ptr(beta), _ptr(ebops_var), _ptr(out), _stream()), 'hgq_ebops_finish_fwd')
    return out


@ebops_finish_fwd.register_fake
def _(ebops, factor, beta, ebops_var):
    return ebops.new_empty(())


@torch.library.custom_op('hgq::ebops_finish_bwd', mutates_args=())
def ebops_finish_bwd(g: Tensor, beta: Tensor, factor: float) -> Tensor:
    _check_f32('g', g)
    d = torch.empty((), dtype=torch.float32, device=g.device)
    _lib.check(_lib.load().hgq_ebops_finish_bwd(_ptr(g), _ptr(beta), factor, _ptr(d), _stream()), 'hgq_ebops_finish_bwd')
    return d


@ebops_finish_bwd.register_fake
def _(g, beta, factor):
    return g.new_empty(())


# ======================================================================================
# autograd pairing
# ======================================================================================
class _Quantize(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, k, i, fb, mode, bw_inner, track):
        y, amax, neg = quantize_fwd(x, k, i, fb, mode, bw_inner, track)
        ctx.save_for_backward(x, k, i, fb)
        ctx.mode, ctx.bw_inner = mode, bw_inner
        ctx.owners = (_owner(i), _owner(fb))
        ctx.mark_non_differentiable(amax, neg)
        ctx.set_materialize_grads(False)
        return y, amax, neg

    @staticmethod
    def backward(ctx, gy, _ga, _gn):
        if gy is None:
            return (None,) * 7
        return _quantize_backward(ctx, gy, ctx.needs_input_grad[0], ctx.needs_input_grad[2], ctx.needs_input_grad[3])


def _quantize_backward(ctx, gy, want_x, want_i, want_fb):
    """Backward of a training-mode quantizer call; ``ctx`` holds (x, k, i, fb), mode, bw_inner and the owners of i, fb.
    Returns the 7-tuple of ``_Quantize``'s inputs."""
    if not (ctx.mode & _lib.MODE_TRAINING):
        raise RuntimeError('hgq quantizer: gradients are defined for the training-mode forward only')
    x, k, i, fb = ctx.saved_tensors
    gy = gy.contiguous()
    # a WRAP quantizer in training mode only rounds: the gradient passes straight through to x
    # and (unless f = b - i) none reaches the integer bits, so the kernel writes neither
    wrap = ((ctx.mode >> 4) & 0xf) == _lib.WRAP
    need_dx = want_x and not wrap
    need_di = want_i and (not wrap or bool(ctx.mode & _lib.MODE_KBI))
    o_i, o_fb = ctx.owners
    if (_SINK['open'] and want_fb and _can_route(o_fb, fb.numel()) and (not need_di or _can_route(o_i, i.numel()))
            and (need_di or not want_i) and quantize_bwd_slices_supported(gy, x, k, i, fb, ctx.bw_inner)):
        # the bit-width gradients go to the optimizer and nowhere else: their slices join the pass's one reduction launch
        dx, ws = quantize_bwd_slices(gy, x, k, i, fb, ctx.mode, ctx.bw_inner, need_dx, need_di)
        dfb, di = torch.empty_like(fb), (torch.empty_like(i) if need_di else None)
        e = fb.new_empty(0)
        _PENDING_REDUCE.append((ws, (dfb.view(-1), di.view(-1) if need_di else e, e), (False, not need_di, True)))
        _route(o_fb, dfb)
        if need_di:
            _route(o_i, di)
        return (gy if wrap else dx) if want_x else None, None, None, None, None, None, None
    dx, di, dfb = quantize_bwd(gy, x, k, i, fb, ctx.mode, ctx.bw_inner, need_dx, need_di)
    if want_x and wrap:
        dx = gy
    if want_i and not need_di:
        di = torch.zeros_like(i)
    return (dx if want_x else None, None, di if want_i else None,
            dfb if want_fb else None, None, None, None)


@torch.library.custom_op('hgq::quantize_fwd_stochastic', mutates_args=())
def quantize_fwd_stochastic(x: Tensor, k: Tensor, i: Tensor, fb: Tensor, mode: int, bw_inner: int, track: bool, seed: int,
                            offset: int) -> tuple[Tensor, Tensor, Tensor]:
    """Training-mode quantizer with stochastic rounding: floor(x * 2^f + u), u a pure function of (seed, offset, element)."""
    _check_f32('x', x), _check_k('k', k), _check_f32('i', i), _check_f32('fb', fb)
    bw = i.numel()
    _need(k.numel() == bw and fb.numel() == bw and bw >= 1 and bw_inner >= 1, 'bit-width operands must have equal sizes')
    y = torch.empty_like(x)
    amax = torch.empty(bw if track else 0, dtype=torch.int32, device=x.device)
    neg = torch.empty(bw if track else 0, dtype=torch.int32, device=x.device)
    m = (_kmode(mode, k) & ~0xf) | _lib.S_RND
    rc = _lib.load().hgq_quantize_fwd_stochastic(_ptr(x), _ptr(k), _ptr(i), _ptr(fb), _ptr(y), _ptr(amax) if track else None,
                                                 _ptr(neg) if track else None, x.numel(), bw, bw_inner, m, seed, offset, _stream())
    _lib.check(rc, 'hgq_quantize_fwd_stochastic')
    return y, amax, neg


@quantize_fwd_stochastic.register_fake
def _(x, k, i, fb, mode, bw_inner, track, seed, offset):
    n = i.numel() if track else 0
    return torch.empty_like(x), x.new_empty(n, dtype=torch.int32), x.new_empty(n, dtype=torch.int32)


@torch.library.custom_op('hgq::quantize_bwd_stochastic', mutates_args=())
def quantize_bwd_stochastic(dy: Tensor, x: Tensor, k: Tensor, i: Tensor, fb: Tensor, mode: int, bw_inner: int, seed: int,
                            offset: int) -> tuple[Tensor, Tensor, Tensor]:
    _check_f32('dy', dy), _check_f32('x', x)
    _need(dy.shape == x.shape, 'dy shape mismatch')
    dx, di, dfb = torch.empty_like(x), torch.empty_like(i), torch.empty_like(fb)
    m = (_kmode(mode, k) & ~0xf) | _lib.S_RND
    rc = _lib.load().hgq_quantize_bwd_stochastic(_ptr(dy), _ptr(x), _ptr(k), _ptr(i), _ptr(fb), _ptr(dx), _ptr(di), _ptr(dfb), x.numel(),
                                                 i.numel(), bw_inner, m, seed, offset, _stream())
    _lib.check(rc, 'hgq_quantize_bwd_stochastic')
    return dx, di, dfb


@quantize_bwd_stochastic.register_fake
def _(dy, x, k, i, fb, mode, bw_inner, seed, offset):
    return torch.empty_like(x), torch.empty_like(i), torch.empty_like(fb)


@torch.library.custom_op('hgq::quantize_fwd_stochastic_at', mutates_args=())
def quantize_fwd_stochastic_at(x: Tensor, k: Tensor, i: Tensor, fb: Tensor, mode: int, bw_inner: int, track: bool, seed: int,
                               offset: int, base: Tensor) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    """``quantize_fwd_stochastic`` whose draw is ``(seed, offset + base[0])`` with ``base`` an int64 counter in device memory;
    the fourth result holds the offset that was used (the backward pass repeats that draw)."""
    _check_f32('x', x), _check_k('k', k), _check_f32('i', i), _check_f32('fb', fb)
    bw = i.numel()
    _need(k.numel() == bw and fb.numel() == bw and bw >= 1 and bw_inner >= 1, 'bit-width operands must have equal sizes')
    _need(base.dtype == torch.int64 and base.numel() == 1 and base.device == x.device, 'base must be one int64 on the device of x')
    y = torch.empty_like(x)
    amax = torch.empty(bw if track else 0, dtype=torch.int32, device=x.device)
    neg = torch.empty(bw if track else 0, dtype=torch.int32, device=x.device)
    used = torch.empty(1, dtype=torch.int64, device=x.device)
    m = (_kmode(mode, k) & ~0xf) | _lib.S_RND
    rc = _lib.load().hgq_quantize_fwd_stochastic_at(_ptr(x), _ptr(k), _ptr(i), _ptr(fb), _ptr(y), _ptr(amax) if track else None,
                                                    _ptr(neg) if track else None, x.numel(), bw, bw_inner, m, seed, offset, _ptr(base),
                                                    _ptr(used), _stream())
    _lib.check(rc, 'hgq_quantize_fwd_stochastic_at')
    return y, amax, neg, used


@quantize_fwd_stochastic_at.register_fake
def _(x, k, i, fb, mode, bw_inner, track, seed, offset, base):
    n = i.numel() if track else 0
    return torch.empty_like(x), x.new_empty(n, dtype=torch.int32), x.new_empty(n, dtype=torch.int32), x.new_empty(1, dtype=torch.int64)


@torch.library.custom_op('hgq::quantize_bwd_stochastic_at', mutates_args=())
def quantize_bwd_stochastic_at(dy: Tensor, x: Tensor, k: Tensor, i: Tensor, fb: Tensor, mode: int, bw_inner: int, seed: int,
                               used: Tensor) -> tuple[Tensor, Tensor, Tensor]:
    _check_f32('dy', dy), _check_f32('x', x)
    _need(dy.shape == x.shape, 'dy shape mismatch')
    _need(used.dtype == torch.int64 and used.numel() == 1 and used.device == x.device, 'used must be one int64 on the device of x')
    dx, di, dfb = torch.empty_like(x), torch.empty_like(i), torch.empty_like(fb)
    m = (_kmode(mode, k) & ~0xf) | _lib.S_RND
    rc = _lib.load().hgq_quantize_bwd_stochastic_at(_ptr(dy), _ptr(x), _ptr(k), _ptr(i), _ptr(fb), _ptr(dx), _ptr(di), _ptr(dfb), x.numel(),
                                                    i.numel(), bw_inner, m, seed, _ptr(used), _stream())
    _lib.check(rc, 'hgq_quantize_bwd_stochastic_at')
    return dx, di, dfb


@quantize_bwd_stochastic_at.register_fake
def _(dy, x, k, i, fb, mode, bw_inner, seed, used):
    return torch.empty_like(x), torch.empty_like(i), torch.empty_like(fb)


@torch.library.custom_op('hgq::counters_advance', mutates_args=('counters',))
def counters_advance(counters: Sequence[Tensor], increments: Sequence[int]) -> None:
    """``counters[j] += increments[j]`` for one-element int64 device tensors, one launch."""
    n = len(counters)
    _need(len(increments) == n, 'one increment per counter')
    if n == 0:
        return
    for c in counters:
        _need(c.dtype == torch.int64 and c.numel() == 1 and c.is_cuda, 'counters are one-element int64 device tensors')
    ptrs = (ctypes.c_void_p * n)(*[c.data_ptr() for c in counters])
    incs = (ctypes.c_uint64 * n)(*[int(v) for v in increments])
    _lib.check(_lib.load().hgq_counters_advance(ptrs, incs, n, _stream()), 'hgq_counters_advance')


# seed generators that drew on the device since their counters were last advanced (hgq2_amd.quantizer.fixed_point_ops)
_SEED_PENDING = []


def advance_seed_generators():
    """Advance the device-side draw counters of the seed generators used since the last call by the number of draws each
    made (one launch).  The outermost layer call of a training step does this before it runs, so a step recorded into a
    HIP graph - counters advanced, then draws at fixed offsets from them - draws anew on every replay."""
    if not _SEED_PENDING:
        return
    gens = [g for g in _SEED_PENDING if g._drawn]
    del _SEED_PENDING[:]
    if gens:
        counters_advance([g._base for g in gens], [g._drawn for g in gens])
        for g in gens:
            g._drawn = 0


class _QuantizeStochasticAt(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, k, i, fb, mode, bw_inner, track, seed, offset, base):
        y, amax, neg, used = quantize_fwd_stochastic_at(x, k, i, fb, mode, bw_inner, track, seed, offset, base)
        ctx.save_for_backward(x, k, i, fb, used)
        ctx.mode, ctx.bw_inner, ctx.seed = mode, bw_inner, seed
        ctx.mark_non_differentiable(amax, neg)
        ctx.set_materialize_grads(False)
        return y, amax, neg

    @staticmethod
    def backward(ctx, gy, _ga, _gn):
        if gy is None:
            return (None,) * 10
        x, k, i, fb, used = ctx.saved_tensors
        dx, di, dfb = quantize_bwd_stochastic_at(gy.contiguous(), x, k, i, fb, ctx.mode, ctx.bw_inner, ctx.seed, used)
        return (dx if ctx.needs_input_grad[0] else None, None, di if ctx.needs_input_grad[2] else None,
                dfb if ctx.needs_input_grad[3] else None, None, None, None, None, None, None)


class _QuantizeStochastic(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, k, i, fb, mode, bw_inner, track, seed, offset):
        y, amax, neg = quantize_fwd_stochastic(x, k, i, fb, mode, bw_inner, track, seed, offset)
        ctx.save_for_backward(x, k, i, fb)
        ctx.mode, ctx.bw_inner, ctx.draw = mode, bw_inner, (seed, offset)
        ctx.mark_non_differentiable(amax, neg)
        ctx.set_materialize_grads(False)
        return y, amax, neg

    @staticmethod
    def backward(ctx, gy, _ga, _gn):
        if gy is None:
            return (None,) * 9
        x, k, i, fb = ctx.saved_tensors
        dx, di, dfb = quantize_bwd_stochastic(gy.contiguous(), x, k, i, fb, ctx.mode, ctx.bw_inner, *ctx.draw)
        return (dx if ctx.needs_input_grad[0] else None, None, di if ctx.needs_input_grad[2] else None,
                dfb if ctx.needs_input_grad[3] else None, None, None, None, None, None)


def quantize_stochastic(x: Tensor, k: Tensor, i: Tensor, fb: Tensor, mode: int, seed: int, offset: int, bw_inner: int = 1,
                        track: bool = False, base: Tensor | None = None):
    """The training-mode quantizer of round modes S_RND / S_RND_CONV; ``(seed, offset)`` names the draw, or
    ``(seed, offset + base[0])`` with a counter in device memory (what a seed generator hands over on the GPU)."""
    _need(bool(mode & _lib.MODE_TRAINING), 'stochastic rounding applies to the training-mode forward only')
    if base is not None:
        return _QuantizeStochasticAt.apply(x.contiguous(), k.contiguous(), i.contiguous(), fb.contiguous(), mode, bw_inner, track,
                                           int(seed), int(offset), base)
    return _QuantizeStochastic.apply(x.contiguous(), k.contiguous(), i.contiguous(), fb.contiguous(), mode, bw_inner, track,
                                     int(seed), int(offset))


class _QuantItem(ctypes.Structure):
    _fields_ = [('x', ctypes.c_void_p), ('k', ctypes.c_void_p), ('i', ctypes.c_void_p), ('fb', ctypes.c_void_p),
                ('y', ctypes.c_void_p), ('n', ctypes.c_int64), ('mode', ctypes.c_int)]


class _QuantGradItem(ctypes.Structure):
    _fields_ = [('dy', ctypes.c_void_p), ('x', ctypes.c_void_p), ('k', ctypes.c_void_p), ('i', ctypes.c_void_p),
                ('fb', ctypes.c_void_p), ('dx', ctypes.c_void_p), ('di', ctypes.c_void_p), ('dfb', ctypes.c_void_p),
                ('n', ctypes.c_int64), ('mode', ctypes.c_int)]


def _check_multi(xs, ks, is_, fbs, modes):
    n = len(xs)
    _need(len(ks) == n and len(is_) == n and len(fbs) == n and len(modes) == n, 'per-quantizer lists differ in length')
    for x, k, i, fb in zip(xs, ks, is_, fbs):
        _check_f32('x', x), _check_k('k', k), _check_f32('i', i), _check_f32('fb', fb)
        _need(k.numel() == x.numel() and i.numel() == x.numel() and fb.numel() == x.numel(),
              'the batched quantizer takes per-element bit-widths (k, i, f of the size of x)')


@torch.library.custom_op('hgq::quantize_fwd_multi', mutates_args=())
def quantize_fwd_multi(xs: Sequence[Tensor], ks: Sequence[Tensor], is_: Sequence[Tensor], fbs: Sequence[Tensor],
                       modes: Sequence[int]) -> list[Tensor]:
    _check_multi(xs, ks, is_, fbs, modes)
    n = len(xs)
    ys = [torch.empty_like(x) for x in xs]
    items = (_QuantItem * max(n, 1))()
    for t in range(n):
        items[t] = _QuantItem(xs[t].data_ptr(), ks[t].data_ptr(), is_[t].data_ptr(), fbs[t].data_ptr(), ys[t].data_ptr(),
                              xs[t].numel(), _kmode(modes[t], ks[t]))
    _lib.check(_lib.load().hgq_quantize_fwd_multi(items, n, _stream()), 'hgq_quantize_fwd_multi')
    return ys


@quantize_fwd_multi.register_fake
def _(xs, ks, is_, fbs, modes):
    return [torch.empty_like(x) for x in xs]


@torch.library.custom_op('hgq::quantize_bwd_multi', mutates_args=())
def quantize_bwd_multi(dys: Sequence[Tensor], xs: Sequence[Tensor], ks: Sequence[Tensor], is_: Sequence[Tensor],
                       fbs: Sequence[Tensor], modes: Sequence[int]) -> list[Tensor]:
    """``dys[t]`` empty: zero upstream gradient.  Returns ``dx_0 .. dx_{n-1}, di_0 .., dfb_0 ..``."""
    _check_multi(xs, ks, is_, fbs, modes)
    n = len(xs)
    _need(len(dys) == n, 'one upstream gradient per quantizer (an empty tensor for none)')
    dxs, dis, dfs = [torch.empty_like(x) for x in xs], [torch.empty_like(i) for i in is_], [torch.empty_like(f) for f in fbs]
    items = (_QuantGradItem * max(n, 1))()
    for t in range(n):
        if dys[t].numel():
            _check_f32('dy', dys[t])
            _need(dys[t].numel() == xs[t].numel(), 'dy and x differ in size')
        items[t] = _QuantGradItem(dys[t].data_ptr() if dys[t].numel() else 0, xs[t].data_ptr(), ks[t].data_ptr(), is_[t].data_ptr(),
                                  fbs[t].data_ptr(), dxs[t].data_ptr(), dis[t].data_ptr(), dfs[t].data_ptr(), xs[t].numel(),
                                  _kmode(modes[t], ks[t]))
    _lib.check(_lib.load().hgq_quantize_bwd_multi(items, n, _stream()), 'hgq_quantize_bwd_multi')
    return dxs + dis + dfs


@quantize_bwd_multi.register_fake
def _(dys, xs, ks, is_, fbs, modes):
    return [torch.empty_like(x) for x in xs] + [torch.empty_like(i) for i in is_] + [torch.empty_like(f) for f in fbs]


class _QuantizeMulti(torch.autograd.Function):
    @staticmethod
    def forward(ctx, n, modes, *tensors):
        xs, ks, is_, fbs = tensors[:n], tensors[n:2 * n], tensors[2 * n:3 * n], tensors[3 * n:]
        ctx.save_for_backward(*tensors)
        ctx.n, ctx.modes = n, modes
        ctx.set_materialize_grads(False)
        return tuple(quantize_fwd_multi(list(xs), list(ks), list(is_), list(fbs), list(modes)))

    @staticmethod
    def backward(ctx, *gys):
        n, t = ctx.n, ctx.saved_tensors
        xs, ks, is_, fbs = t[:n], t[n:2 * n], t[2 * n:3 * n], t[3 * n:]
        for mode in ctx.modes:
            if not (mode & _lib.MODE_TRAINING):
                raise RuntimeError('hgq quantizer: gradients are defined for the training-mode forward only')
        dys = [x.new_empty(0) if g is None else g.contiguous() for g, x in zip(gys, xs)]
        out = _reduce_and_quantize_bwd(dys, xs, ks, is_, fbs, ctx.modes)
        if out is None:
            flush_reductions()
            out = quantize_bwd_multi(dys, list(xs), list(ks), list(is_), list(fbs), list(ctx.modes))
        need = ctx.needs_input_grad[2:]
        grads = list(out[:n]) + [None] * n + list(out[n:])
        return (None, None) + tuple(g if need[j] else None for j, g in enumerate(grads))


def quantize_multi(xs, ks, is_, fbs, modes):
    """Several quantizers with per-element bit-widths in one launch each way; returns the quantized tensors."""
    n = len(xs)
    flat = [t.contiguous() for group in (xs, ks, is_, fbs) for t in group]
    return _QuantizeMulti.apply(n, tuple(int(m) for m in modes), *flat)


def quantize(x: Tensor, k: Tensor, i: Tensor, fb: Tensor, mode: int, bw_inner: int = 1, track: bool = False):
    """Fixed-point quantizer.  Returns ``(y, amax_bits, anyneg)``; the last two are empty unless ``track``."""
    return _Quantize.apply(x.contiguous(), k.contiguous(), i.contiguous(), fb.contiguous(), mode, bw_inner, track)


def wrap_track_i_(amax, i_var, fb, decay, mode, c_lo=float('-inf'), c_hi=float('inf'), anyneg=None, k_var=None):
    """In-place integer-bit tracking; ``amax`` is [m] or [n_parts, m]."""
    m = i_var.numel()
    n_parts = amax.numel() // m
    if (_DEFER['dense_ebops'] or _DEFER['late']) and _reads_queued(i_var):
        flush_deferred()  # a queued EBOPs estimate reads these integer bits as they stand now
    if (_DEFER['depth'] > 0 and anyneg is None and k_var is None and not (mode & (_lib.MODE_KBI | _lib.MODE_TRACING))
            and c_lo == float('-inf') and c_hi == float('inf')):
        # a KIF quantizer's training-mode update (its own forward does not read the integer bits): joins the other
        # quantizers' updates of this model call in one launch, ahead of the first reader
        _DEFER['tracks'].append((amax, i_var, fb, decay, mode))
        return
    touch_state()
    _keep((amax, anyneg))
    empty_i = amax.new_empty(0)
    empty_k = torch.empty(0, dtype=torch.uint8, device=amax.device)
    wrap_track_i_op(amax, anyneg if anyneg is not None else empty_i, n_parts, i_var, fb,
                    k_var if k_var is not None else empty_k, float(decay), float(c_lo), float(c_hi), mode)


FUSED_BWD_MAX = 64  # hgq_qdense_bwd covers K <= 64 and N <= 64


class _QDense(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, k_in, i_in, f_in, qw, qb, act, mode, bw_rows, track):
        y, amax = qdense_fwd(x, k_in, i_in, f_in, qw, qb, act, mode, bw_rows, track)
        ctx.f_owner = _owner(f_in)
        ctx.save_for_backward(x, f_in, qw, y)
        ctx.has_bias = qb.numel() > 0
        # both operands were handed out once by the model-wide weight-quantizer launch: their only reader is its backward
        ctx.defer = getattr(qw, '_hgq_single_use', False) and (qb.numel() == 0 or getattr(qb, '_hgq_single_use', False))
        ctx.act, ctx.mode, ctx.bw_rows, ctx.f_shape = act, mode, bw_rows, f_in.shape
        ctx.mark_non_differentiable(amax)
        ctx.set_materialize_grads(False)
        return y, amax

    @staticmethod
    def backward(ctx, gy, _ga):
        if gy is None:
            return (None,) * 10
        x, f_in, qw, y = ctx.saved_tensors
        if ctx.defer and _SINK['open'] and (ctx.bw_rows == 0 or _can_route(ctx.f_owner, ctx.bw_rows * x.shape[1])):
            # the kernel / bias gradients are first read by the backward of the prefetched quantizers and the bit-width
            # gradient by the optimizer: their slice reduction joins those of the other layers
            dx, ws = qdense_bwd_slices(gy.contiguous(), y, x, f_in, qw, ctx.has_bias, ctx.act, ctx.mode, ctx.bw_rows)
            K, N = qw.shape
            dqw, dqb, df = torch.empty_like(qw), x.new_empty(N), x.new_empty(ctx.bw_rows * K)
            _PENDING_REDUCE.append((ws, (dqw, dqb, df), (False, not ctx.has_bias, False)))
        else:
            dx, dqw, dqb, df = qdense_bwd(gy.contiguous(), y, x, f_in, qw, ctx.has_bias, ctx.act, ctx.mode, ctx.bw_rows)
        df = _route(ctx.f_owner, df) if ctx.bw_rows > 0 else None
        return (dx, None, None, df.view(ctx.f_shape) if df is not None else None, dqw, dqb if ctx.has_bias else None,
                None, None, None, None)


def qdense(x2d, k_in, i_in, f_in, qw, qb, act: int, mode: int, bw_rows: int, track: bool):
    """y = act(q_in(x) @ qw + qb) on a [rows, K] view; returns ``(y, amax slices)``."""
    empty = x2d.new_empty(0)
    return _QDense.apply(x2d, k_in if k_in is not None else empty, i_in if i_in is not None else empty,
                         f_in if f_in is not None else empty, qw, qb if qb is not None else empty, act, mode, bw_rows, track)


class _QDenseMean(torch.autograd.Function):
    """``_QDense`` followed by a mean over groups of ``mean_rows`` rows, as one launch each way: returns
    ``(group means, amax slices)``; the contraction's own output is never written (the backward pass reads a bit per output,
    the ReLU mask, instead)."""

    @staticmethod
    def forward(ctx, x, k_in, f_in, qw, qb, act, mode, bw_rows, mean_rows):
        mask, ymean, amax = qdense_fwd_mean(x, k_in, f_in, qw, qb, act, mode, bw_rows, mean_rows)
        ctx.f_owner = _owner(f_in)
        ctx.save_for_backward(x, f_in, qw, mask)
        ctx.has_bias = qb.numel() > 0
        ctx.defer = getattr(qw, '_hgq_single_use', False) and (qb.numel() == 0 or getattr(qb, '_hgq_single_use', False))
        ctx.act, ctx.mode, ctx.bw_rows, ctx.f_shape, ctx.mean_rows = act, _kmode(mode, k_in) if bw_rows > 0 else mode, bw_rows, f_in.shape, mean_rows
        ctx.mark_non_differentiable(amax)
        ctx.set_materialize_grads(False)
        return ymean, amax

    @staticmethod
    def backward(ctx, gm, _ga):
        if gm is None:
            return (None,) * 9
        x, f_in, qw, mask = ctx.saved_tensors
        if ctx.defer and _SINK['open'] and (ctx.bw_rows == 0 or _can_route(ctx.f_owner, ctx.bw_rows * x.shape[1])):
            dx, ws = qdense_bwd_mean_slices(gm.contiguous(), mask, x, f_in, qw, ctx.has_bias, ctx.act, ctx.mode, ctx.bw_rows, ctx.mean_rows)
            K, N = qw.shape
            dqw, dqb, df = torch.empty_like(qw), x.new_empty(N), x.new_empty(ctx.bw_rows * K)
            _PENDING_REDUCE.append((ws, (dqw, dqb, df), (False, not ctx.has_bias, False)))
        else:
            dx, dqw, dqb, df = qdense_bwd_mean(gm.contiguous(), mask, x, f_in, qw, ctx.has_bias, ctx.act, ctx.mode, ctx.bw_rows, ctx.mean_rows)
        df = _route(ctx.f_owner, df) if ctx.bw_rows > 0 else None
        return (dx, None, df.view(ctx.f_shape) if df is not None else None, dqw, dqb if ctx.has_bias else None, None, None, None, None)


def qdense_mean_supported(rows: int, K: int, N: int, bw_rows: int, mean_rows: int, mode: int) -> bool:
    """Whether ``qdense_mean`` covers the shape and the input quantizer's mode."""
    return bool(_lib.load().hgq_qdense_fwd_mean_supported(rows, K, N, bw_rows, mean_rows, mode))


def qdense_mean(x2d, k_in, f_in, qw, qb, act: int, mode: int, bw_rows: int, mean_rows: int):
    """Group means of ``act(q_in(x) @ qw + qb)`` over ``mean_rows`` consecutive rows of a [rows, K] view; returns
    ``(means [rows / mean_rows, N], amax slices)``."""
    empty = x2d.new_empty(0)
    return _QDenseMean.apply(x2d, k_in if k_in is not None else empty, f_in if f_in is not None else empty, qw,
                             qb if qb is not None else empty, act, mode, bw_rows, mean_rows)


class _QDenseOQ(torch.autograd.Function):
    """``_QDense`` whose forward kernel also runs the layer's output quantizer: returns ``(y, yq, amax, oamax)`` with the
    gradient of ``_QDense`` on ``y``; ``yq`` carries no gradient here - ``_QuantizeGiven`` ties it to ``y``."""

    @staticmethod
    def forward(ctx, x, k_in, f_in, qw, qb, k_out, f_out, act, mode, mode_out, bw_rows, bw_rows_out):
        y, yq, amax, oamax = qdense_fwd_oq(x, k_in, f_in, qw, qb, k_out, f_out, act, mode, mode_out, bw_rows, bw_rows_out)
        ctx.f_owner = _owner(f_in)
        ctx.save_for_backward(x, f_in, qw, y)
        ctx.has_bias = qb.numel() > 0
        ctx.defer = getattr(qw, '_hgq_single_use', False) and (qb.numel() == 0 or getattr(qb, '_hgq_single_use', False))
        ctx.act, ctx.mode, ctx.bw_rows, ctx.f_shape = act, _kmode(mode, k_in), bw_rows, f_in.shape
        ctx.mark_non_differentiable(yq, amax, oamax)
        ctx.set_materialize_grads(False)
        return y, yq, amax, oamax

    @staticmethod
    def backward(ctx, gy, _gq, _ga, _go):
        if gy is None:
            return (None,) * 12
        dx, _, _, df, dqw, dqb, _, _, _, _ = _QDense.backward(ctx, gy, None)
        return dx, None, df, dqw, dqb, None, None, None, None, None, None, None


class _QuantizeGiven(torch.autograd.Function):
    """A quantizer call whose forward another kernel has already run (``yq`` = the quantized ``x``): hands ``yq`` on with
    the backward of ``_Quantize``."""

    @staticmethod
    def forward(ctx, x, yq, k, i, fb, mode, bw_inner):
        ctx.save_for_backward(x, k, i, fb)
        ctx.mode, ctx.bw_inner = mode, bw_inner
        ctx.owners = (_owner(i), _owner(fb))
        ctx.set_materialize_grads(False)
        return yq.view_as(yq)

    @staticmethod
    def backward(ctx, gy):
        if gy is None:
            return (None,) * 7
        dx, _, di, dfb, _, _, _ = _quantize_backward(ctx, gy, ctx.needs_input_grad[0], ctx.needs_input_grad[3], ctx.needs_input_grad[4])
        return dx, None, None, di, dfb, None, None


def qdense_oq(x2d, k_in, f_in, qw, qb, k_out, i_out, f_out, act: int, mode: int, mode_out: int, bw_rows: int, bw_rows_out: int):
    """``q_out(act(q_in(x) @ qw + qb))`` on a [rows, K] view with both quantizers (KIF, WRAP, training mode: they only
    round) inside the contraction kernel; returns ``(yq, amax slices of the input quantizer, amax slices of the output
    quantizer)``.  The backward is the output quantizer's own (its fractional-bit gradient from the stored ``y``; the data
    gradient passes unchanged) followed by the contraction's."""
    empty = x2d.new_empty(0)
    y, yq, amax, oamax = _QDenseOQ.apply(x2d, k_in, f_in, qw, qb if qb is not None else empty, k_out, f_out, act, mode, mode_out,
                                         bw_rows, bw_rows_out)
    yq = _QuantizeGiven.apply(y, yq, k_out, i_out, f_out, _kmode(mode_out, k_out), 1)
    return yq, amax, oamax


class _DenseEbops(torch.autograd.Function):
    @staticmethod
    def forward(ctx, i_in, f_in, b_ker, b_bias, amax, decay, beta, k_in, k_ker, k_bias, ebops_var, P, K, N, scale, bias_size,
                mode_in, mode_ker, mode_bias, owners):  # scale = (par_factor, n_parallel, ebops_factor)
        ctx.owners = owners
        _keep((amax,))
        if _DEFER['depth'] > 0:  # inside a model call: queued, launched with the other layers' when the call returns
            op = _dense_ebops_queue
        else:
            op = dense_ebops_track_op if amax.numel() else dense_ebops_op
        ebops, term, g = op(amax, decay, beta, k_in, i_in, f_in, k_ker, b_ker, k_bias, b_bias, ebops_var, P, K, N,
                                        *scale, bias_size, mode_in, mode_ker, mode_bias)
        ctx.g = g  # kept as a plain attribute: a queued call fills it after this function has returned
        ctx.has_beta = beta.numel() > 0
        ctx.sizes = (P * K, K * N, b_bias.numel())
        ctx.kbi_in = bool(mode_in & _lib.MODE_KBI)
        ctx.shapes = (i_in.shape, f_in.shape, b_ker.shape, b_bias.shape)
        ctx.set_materialize_grads(False)
        if ctx.has_beta:
            ctx.mark_non_differentiable(ebops)
        else:
            ctx.mark_non_differentiable(term)
        return ebops, term

    @staticmethod
    def backward(ctx, g_ebops, g_term):
        g = ctx.g
        up = g_term if ctx.has_beta else g_ebops
        if up is None:
            return (None,) * 20
        n_f, n_k, n_b = ctx.sizes
        s_i, s_f, s_k, s_b = ctx.shapes
        want_i = ctx.needs_input_grad[0] and not ctx.kbi_in
        if _SINK['open'] and ctx.owners is not None:
            # the pieces stay as the kernel left them (for a unit upstream gradient) and go to the optimizer with `up`
            o_i, o_f, o_k, o_b = ctx.owners
            pieces = [(o_f, g[:n_f]), (o_k, g[n_f:n_f + n_k])]
            if want_i:
                pieces.append((o_i, g[:n_f]))
            if n_b:
                pieces.append((o_b, g[n_f + n_k:]))
            if all(_parkable(o) for o, _ in pieces):
                for o, piece in pieces:
                    _stash_side(o, up, piece)
                return (None,) * 20
        join_side()  # the kernel that fills `g` may have run on the second stream
        grads = g if _is_unit(up) else up * g
        gf = grads[:n_f]
        gi = gf.view(s_i) if want_i else None
        return (gi, gf.view(s_f), grads[n_f:n_f + n_k].view(s_k), grads[n_f + n_k:].view(s_b) if n_b else None) + (None,) * 16


def dense_ebops(k_in, i_in, f_in, k_ker, b_ker, k_bias, b_bias, P, K, N, par_factor, n_parallel, ebops_factor, bias_size, mode_in,
                mode_ker, mode_bias, amax=None, decay=0.0, beta=None, ebops_var=None, owners=None):
    """EBOPs of a dense contraction, scaled as ``sum * par_factor / n_parallel * ebops_factor`` left to right in fp32
    (reference src/hgq/layers/core/dense.py:80, base.py:102).  Returns ``(ebops, ebops * beta)``: with ``beta`` the second
    carries the gradient (and the first is a plain value), without it the first does.  With
    ``amax`` the input quantizer's integer bits are tracked in place first; with ``ebops_var`` the
    uint32 variable is assigned.  ``owners`` = the variables behind ``(i_in, f_in, b_ker, b_bias)``: with the gradient
    sink open their gradient pieces are left on them instead of going back through autograd."""
    dev = f_in.device
    e_f = torch.empty(0, dtype=torch.float32, device=dev)
    e_i = torch.empty(0, dtype=torch.int32, device=dev)
    e_k = torch.empty(0, dtype=torch.uint8, device=dev)
    return _DenseEbops.apply(i_in, f_in, b_ker, b_bias if b_bias is not None else e_f, amax if amax is not None else e_i,
                             float(decay), beta if beta is not None else e_f, k_in, k_ker,
                             k_bias if k_bias is not None else e_k, ebops_var if ebops_var is not None else e_i, P, K, N,
                             (float(par_factor), float(n_parallel), float(ebops_factor)), float(bias_size), mode_in, mode_ker,
                             mode_bias, owners)


class _QSoftmax(torch.autograd.Function):
    """Arguments after the scalars: k, i, fb of exp_iq, exp_oq, inv_iq, inv_oq, oq (15 tensors, empty = absent)."""

    @staticmethod
    def forward(ctx, x, modes, input_scaler, eps, track_mask, *qvars):
        ks, is_, fbs = list(qvars[0::3]), list(qvars[1::3]), list(qvars[2::3])
        y, a1, a3, ao = qsoftmax_fwd(x, ks, is_, fbs, list(modes), input_scaler, eps, track_mask)
        ctx.save_for_backward(x, *qvars)
        ctx.modes, ctx.input_scaler, ctx.eps = tuple(modes), input_scaler, eps
        ctx.mark_non_differentiable(a1, a3, ao)
        ctx.set_materialize_grads(False)
        return y, a1, a3, ao

    @staticmethod
    def backward(ctx, gy, *_unused):
        n_in = 5 + 15
        if gy is None:
            return (None,) * n_in
        x, *qvars = ctx.saved_tensors
        ks, is_, fbs = list(qvars[0::3]), list(qvars[1::3]), list(qvars[2::3])
        dx, g_shared, g_oi, g_of = qsoftmax_bwd(gy.contiguous(), x, ks, is_, fbs, list(ctx.modes), ctx.input_scaler, ctx.eps)
        grads = [dx if ctx.needs_input_grad[0] else None, None, None, None, None]
        for n in range(5):
            gi = g_shared[2 * n] if n < 4 else g_oi
            gf = g_shared[2 * n + 1] if n < 4 else g_of
            present = ks[n].numel() > 0
            base = 5 + 3 * n
            grads.append(None)
            grads.append(gi.view(is_[n].shape) if present and ctx.needs_input_grad[base + 1] else None)
            grads.append(gf.view(fbs[n].shape) if present and ctx.needs_input_grad[base + 2] else None)
        return tuple(grads)


def qsoftmax(x: Tensor, quantizers, input_scaler: float, eps: float, track_mask: int = 0):
    """Table-driven softmax over the last axis.  ``quantizers`` = five entries (exp_iq, exp_oq, inv_iq,
    inv_oq, oq), each ``None`` or ``(k, i, fb, mode)``.  Returns ``(y, amax_exp_iq, amax_inv_iq, amax_oq)``."""
    e_f = x.new_empty(0)
    e_k = torch.empty(0, dtype=torch.uint8, device=x.device)
    flat, modes = [], []
    for q in quantizers:
        if q is None:
            flat += [e_k, e_f, e_f]
            modes.append(0)
        else:
            k, i, fb, mode = q
            flat += [k.contiguous(), i.contiguous(), fb.contiguous()]
            modes.append(int(mode))
    return _QSoftmax.apply(x.contiguous(), tuple(modes), float(input_scaler), float(eps), int(track_mask), *flat)


class _QAttention(torch.autograd.Function):
    """Arguments after the scalars: k, i, fb of exp_iq, exp_oq, inv_iq, inv_oq, oq (15 tensors, empty = absent)."""

    @staticmethod
    def forward(ctx, q, k, v, modes, input_scaler, eps, track_mask, mask, causal, *qvars):
        ks, is_, fbs = list(qvars[0::3]), list(qvars[1::3]), list(qvars[2::3])
        out, a1, a3, ao = qattention_fwd(q, k, v, ks, is_, fbs, list(modes), input_scaler, eps, track_mask, mask, causal)
        ctx.save_for_backward(q, k, v, mask, *qvars)
        ctx.modes, ctx.input_scaler, ctx.eps, ctx.causal = tuple(modes), input_scaler, eps, causal
        ctx.mark_non_differentiable(a1, a3, ao)
        ctx.set_materialize_grads(False)
        return out, a1, a3, ao

    @staticmethod
    def backward(ctx, gout, *_unused):
        n_in = 9 + 15
        if gout is None:
            return (None,) * n_in
        q, k, v, mask, *qvars = ctx.saved_tensors
        ks, is_, fbs = list(qvars[0::3]), list(qvars[1::3]), list(qvars[2::3])
        dq, dk, dv, g_shared, g_oi, g_of = qattention_bwd(gout.contiguous(), q, k, v, ks, is_, fbs, list(ctx.modes),
                                                          ctx.input_scaler, ctx.eps, mask, ctx.causal)
        need = ctx.needs_input_grad
        grads = [dq if need[0] else None, dk if need[1] else None, dv if need[2] else None, None, None, None, None, None, None]
        for n in range(5):
            gi = g_shared[2 * n] if n < 4 else g_oi
            gf = g_shared[2 * n + 1] if n < 4 else g_of
            present = ks[n].numel() > 0
            base = 9 + 3 * n
            grads.append(None)
            grads.append(gi.view(is_[n].shape) if present and need[base + 1] else None)
            grads.append(gf.view(fbs[n].shape) if present and need[base + 2] else None)
        return tuple(grads)


def qattention(q: Tensor, k: Tensor, v: Tensor, quantizers, input_scaler: float, eps: float, track_mask: int = 0, mask=None,
               causal: bool = False):
    """``combine(qsoftmax(scores(q, k)), v)`` without materialising scores or probabilities.  ``quantizers`` as for
    ``qsoftmax``.  ``mask``: boolean ``[1 or B, T, S]`` (False = masked out, shared by the heads) or None; ``causal``: key
    positions beyond the query position are masked as well.  Returns ``(out, amax_exp_iq, amax_inv_iq, amax_oq)``."""
    if mask is None:
        mask = torch.empty(0, dtype=torch.uint8, device=q.device)
    else:
        mask = mask.to(torch.uint8).contiguous()
    e_f = q.new_empty(0)
    e_k = torch.empty(0, dtype=torch.uint8, device=q.device)
    flat, modes = [], []
    for qz in quantizers:
        if qz is None:
            flat += [e_k, e_f, e_f]
            modes.append(0)
        else:
            kk, i, fb, mode = qz
            flat += [kk.contiguous(), i.contiguous(), fb.contiguous()]
            modes.append(int(mode))
    return _QAttention.apply(q.contiguous(), k.contiguous(), v.contiguous(), tuple(modes), float(input_scaler), float(eps),
                             int(track_mask), mask, bool(causal), *flat)


class _Conv2D(torch.autograd.Function):
    @staticmethod
    def forward(ctx, xq, qw, qb, geom, act):
        y = conv2d_fwd(xq, qw, qb, list(geom), act)
        ctx.save_for_backward(xq, qw, y)
        ctx.geom, ctx.act, ctx.has_bias = tuple(geom), act, qb.numel() > 0
        # both operands were handed out once by the model-wide weight-quantizer launch: their only reader is its backward
        ctx.defer = getattr(qw, '_hgq_single_use', False) and (qb.numel() == 0 or getattr(qb, '_hgq_single_use', False))
        return y

    @staticmethod
    def backward(ctx, gy):
        xq, qw, y = ctx.saved_tensors
        if ctx.defer and _SINK['open']:
            # kernel and bias gradient are first read by the backward of the prefetched quantizers: their slices join the
            # pass's one reduction launch
            dx, ws = conv2d_bwd_slices(gy.contiguous(), y, xq, qw, list(ctx.geom), ctx.act, ctx.needs_input_grad[0])
            dqw, dqb = torch.empty_like(qw), xq.new_empty(qw.shape[-1])
            _PENDING_REDUCE.append((ws, (dqw.view(-1), dqb, xq.new_empty(0)), (False, not ctx.has_bias, True)))
        else:
            dx, dqw, dqb = conv2d_bwd(gy.contiguous(), y, xq, qw, list(ctx.geom), ctx.act, ctx.needs_input_grad[0], ctx.has_bias)
        return (dx if ctx.needs_input_grad[0] else None, dqw, dqb if ctx.has_bias else None, None, None)


class _Conv2DMaxPool(torch.autograd.Function):
    """Convolution and the 2 x 2 maximum pooling that is its only reader as one node: the unpooled output is never
    written; a byte per window and filter (where the maximum sat, whether it was positive) is saved for the backward
    pass, which forms the unpooled gradient from the pooled one while it stages its tiles."""

    @staticmethod
    def forward(ctx, xq, qw, qb, geom, act):
        y, yp = conv2d_maxpool_fwd_coded(xq, qw, qb, list(geom), act)
        ctx.save_for_backward(xq, qw, y)
        ctx.geom, ctx.act, ctx.has_bias = tuple(geom), act, qb.numel() > 0
        ctx.defer = getattr(qw, '_hgq_single_use', False) and (qb.numel() == 0 or getattr(qb, '_hgq_single_use', False))
        return yp

    @staticmethod
    def backward(ctx, gyp):
        xq, qw, y = ctx.saved_tensors
        need_dx = ctx.needs_input_grad[0]
        if ctx.defer and _SINK['open']:  # as in _Conv2D: the slices join the pass's one reduction launch
            dx, ws = conv2d_maxpool_bwd_coded(gyp.contiguous(), y, xq, qw, list(ctx.geom), ctx.act, need_dx, False)
            dqw, dqb = torch.empty_like(qw), xq.new_empty(qw.shape[-1])
            _PENDING_REDUCE.append((ws, (dqw.view(-1), dqb, xq.new_empty(0)), (False, not ctx.has_bias, True)))
        else:
            dx, flat = conv2d_maxpool_bwd_coded(gyp.contiguous(), y, xq, qw, list(ctx.geom), ctx.act, need_dx, True)
            dqw, dqb = flat[:qw.numel()].view(qw.shape), flat[qw.numel():]
        return (dx if need_dx else None, dqw, dqb if ctx.has_bias else None, None, None)


def conv2d(xq: Tensor, qw: Tensor, qb, strides=(1, 1), padding='valid', dilation=(1, 1), act: int = 0, maxpool2: bool = False) -> Tensor:
    """``act(conv2d(xq, qw) + qb)`` for a channels-last input [B, H, W, C] and an HWIO kernel; 'same'
    padding puts the odd pad after the last row / column, as Keras / TensorFlow do.  ``maxpool2``: followed by a 2 x 2
    maximum pooling of stride 2 without padding, for shapes ``conv2d_maxpool_supported`` accepts."""
    _need(qw.shape[2] == xq.shape[3], f'kernel has {qw.shape[2]} input channels, input has {xq.shape[3]}')
    geom = conv_geometry(tuple(xq.shape), tuple(qw.shape), strides, padding, dilation)
    if maxpool2:
        _need(conv2d_maxpool_supported(geom, qw.shape[-1]), 'convolution + pooling in one node: shape not supported')
        return _Conv2DMaxPool.apply(xq.contiguous(), qw.contiguous(), qb.contiguous() if qb is not None else xq.new_empty(0), geom, act)
    return _Conv2D.apply(xq.contiguous(), qw.contiguous(), qb.contiguous() if qb is not None else xq.new_empty(0), geom, act)


def matmul_bias_act(x2d: Tensor, qw: Tensor, qb, act: int = 0) -> Tensor:
    """``act(x2d @ qw + qb)`` for any K, N: the 1 x 1 case of the implicit-GEMM kernels."""
    rows, K = x2d.shape
    N = qw.shape[1]
    geom = (rows, 1, 1, K, 1, 1, 1, 1, 0, 0, 1, 1, 1, 1)
    w4 = qw.contiguous().view(1, 1, K, N)
    if getattr(qw, '_hgq_single_use', False) and w4._base is qw:
        w4._hgq_single_use = True  # a view's gradient goes back through the view unread: the one-reader mark holds for it
    y = _Conv2D.apply(x2d.contiguous(), w4, qb.contiguous() if qb is not None else x2d.new_empty(0), geom, act)
    return y.view(rows, N)


class _ColMoments(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        mean, meansq = col_moments_fwd(x)
        ctx.save_for_backward(x)
        return mean, meansq

    @staticmethod
    def backward(ctx, gm, gs):
        (x,) = ctx.saved_tensors
        gm = torch.zeros(x.shape[1], device=x.device) if gm is None else gm.contiguous()
        gs = torch.zeros(x.shape[1], device=x.device) if gs is None else gs.contiguous()
        return col_moments_bwd(x, gm, gs)


def col_moments(x2d: Tensor):
    """``(mean(x, 0), mean(x * x, 0))`` of a [rows, N] matrix in one pass."""
    return _ColMoments.apply(x2d.contiguous())


class _DenseMoments(torch.autograd.Function):
    """``chain``: the input is also returned, as the third output, for its other consumer (the output contraction of
    the same layer); the gradient that comes back through it is added while this backward writes dx, instead of in an
    accumulation pass of its own."""

    @staticmethod
    def forward(ctx, x, w, f_in, bw_rows, mode, chain):
        ctx.save_for_backward(x, w, f_in)
        ctx.quant = (bw_rows, mode)
        ctx.owners = (_owner(w), _owner(f_in))
        mean, meansq = dense_moments_fwd(x, w, f_in, bw_rows, mode)
        return (mean, meansq, x) if chain else (mean, meansq)

    @staticmethod
    def backward(ctx, dmean, dmeansq, dx_chain=None):
        x, w, f_in = ctx.saved_tensors
        bw_rows, mode = ctx.quant
        zero = x.new_zeros(w.shape[1]) if (dmean is None or dmeansq is None) else None
        # without a consumer of dx (an input that needs no gradient) the chained gradient is not read either
        dx_add = x.new_empty(0) if dx_chain is None or not ctx.needs_input_grad[0] else dx_chain.contiguous()
        o_w, o_f = ctx.owners
        gm, gs = dmean.contiguous() if dmean is not None else zero, dmeansq.contiguous() if dmeansq is not None else zero
        if _SINK['open'] and _can_route(o_w, w.numel()) and (not bw_rows or _can_route(o_f, f_in.numel())):
            # kernel and fractional-bit gradient go to the optimizer and nowhere else: their slices join the pass's one reduction
            dx, ws = dense_moments_bwd_slices(x, w, f_in, bw_rows, mode, gm, gs, dx_add)
            dw, df = torch.empty_like(w), x.new_empty(bw_rows * x.shape[1])
            _PENDING_REDUCE.append((ws, (dw.view(-1), x.new_empty(w.shape[1]), df), (False, True, not bw_rows)))
        else:
            dx, dw, df = dense_moments_bwd(x, w, f_in, bw_rows, mode, gm, gs, dx_add)
        dw = _route(o_w, dw)
        df = _route(o_f, df) if bw_rows else None
        return dx, dw, (df.view(f_in.shape) if df is not None else None), None, None, None


def dense_moments(x2d: Tensor, w2d: Tensor, quant=None, chain=False):
    """``(mean(z, 0), mean(z * z, 0))`` of ``z = q(x2d) @ w2d`` without materialising ``z`` (nor ``q(x2d)``).
    ``quant`` = ``(f_in, bw_rows, mode)``: the raw fractional bits of a training-mode WRAP input quantizer laid out as
    a ``[bw_rows, K]`` table; ``None``: ``x2d`` is contracted as it is.  ``chain``: a third result, ``x2d`` again, to be
    used by the caller instead of ``x2d`` from here on (see ``_DenseMoments``)."""
    if quant is None:
        return _DenseMoments.apply(x2d.contiguous(), w2d.contiguous(), x2d.new_empty(0), 0, 0, chain)
    f_in, bw_rows, mode = quant
    return _DenseMoments.apply(x2d.contiguous(), w2d.contiguous(), f_in.contiguous(), int(bw_rows), int(mode), chain)


class _BnFold(torch.autograd.Function):
    @staticmethod
    def forward(ctx, w, bias, gamma, mean, second, is_meansq, eps, moving_mean, moving_var, momentum):
        ctx.save_for_backward(w, gamma, mean, second)
        ctx.cfg = (is_meansq, eps)
        ctx.w_owner = _owner(w)
        return bn_fold_fwd(w, bias, gamma, mean, second, is_meansq, eps, moving_mean, moving_var, momentum)

    @staticmethod
    def backward(ctx, d_fw, d_fb):
        w, gamma, mean, second = ctx.saved_tensors
        is_meansq, eps = ctx.cfg
        dw, dbias, dgamma, dmean, dsecond = bn_fold_bwd(w, gamma, mean, second, is_meansq, eps, d_fw.contiguous(), d_fb.contiguous())
        return _route(ctx.w_owner, dw), dbias, (dgamma if gamma.numel() else None), dmean, dsecond, None, None, None, None, None


class _BnFoldQuant(torch.autograd.Function):
    """``_BnFold`` and the kernel / bias quantizers behind it, one launch each way."""

    @staticmethod
    def forward(ctx, w, bias, gamma, mean, second, is_meansq, eps, moving_mean, moving_var, momentum, modes, k_k, i_k, fb_k, k_b, i_b, fb_b):
        ctx.save_for_backward(w, bias, gamma, mean, second, k_k, i_k, fb_k, k_b, i_b, fb_b)
        ctx.cfg = (is_meansq, eps, modes)
        ctx.w_owner = _owner(w)
        ctx.set_materialize_grads(False)
        return bn_fold_quant_fwd(w, bias, gamma, mean, second, is_meansq, eps, moving_mean, moving_var, momentum, [k_k, i_k, fb_k],
                                 [k_b, i_b, fb_b], list(modes))

    @staticmethod
    def backward(ctx, d_qw, d_qb):
        flush_reductions()  # the kernel / bias gradient may still be slices of the contraction's backward
        w, bias, gamma, mean, second, k_k, i_k, fb_k, k_b, i_b, fb_b = ctx.saved_tensors
        is_meansq, eps, modes = ctx.cfg
        d_qw = torch.zeros_like(w) if d_qw is None else d_qw.contiguous()
        d_qb = torch.zeros_like(bias) if d_qb is None else d_qb.contiguous()
        dw, dbias, dgamma, dmean, dsecond, di_k, dfb_k, di_b, dfb_b = bn_fold_quant_bwd(
            w, bias, gamma, mean, second, is_meansq, eps, d_qw.view(w.shape), d_qb.view(bias.shape), [k_k, i_k, fb_k], [k_b, i_b, fb_b],
            list(modes))
        need = ctx.needs_input_grad
        return (_route(ctx.w_owner, dw), dbias, (dgamma if gamma.numel() else None), dmean, dsecond, None, None, None, None, None, None,
                None, di_k.view(i_k.shape) if need[12] else None, dfb_k.view(fb_k.shape) if need[13] else None,
                None, di_b.view(i_b.shape) if need[15] else None, dfb_b.view(fb_b.shape) if need[16] else None)


def bn_fold_quant(w2d: Tensor, bias: Tensor, gamma, mean: Tensor, second: Tensor, is_meansq: bool, eps: float, moving_mean, moving_var,
                  momentum: float, qk, qb):
    """``(q_k(w s), q_b(bias - mean s))``: :func:`bn_fold` and the two quantizers ``qk`` / ``qb`` = ``(k, i, fb, mode)`` (flat
    raw variables of training-mode quantizers with per-element bit-widths and no trackers) in one launch each way."""
    empty = w2d.new_empty(0)
    return _BnFoldQuant.apply(w2d.contiguous(), bias.contiguous(), gamma.contiguous() if gamma is not None else empty, mean.contiguous(),
                              second.contiguous(), bool(is_meansq), float(eps), moving_mean if moving_mean is not None else empty,
                              moving_var if moving_var is not None else empty, float(momentum), (int(qk[3]), int(qb[3])),
                              qk[0], qk[1], qk[2], qb[0], qb[1], qb[2])


def bn_fold(w2d: Tensor, bias: Tensor, gamma, mean: Tensor, second: Tensor, is_meansq: bool, eps: float, moving_mean=None,
            moving_var=None, momentum: float = 0.0):
    """Batch-norm folding ``(w * s, bias - mean * s)`` with ``s = gamma / sqrt(var + eps)`` for a ``[K, N]`` kernel
    normalised over its outputs; ``second`` is the mean of squares (``is_meansq``) or the variance.  Moving statistics,
    when given, are updated in place with ``momentum``."""
    empty = w2d.new_empty(0)
    return _BnFold.apply(w2d.contiguous(), bias.contiguous(), gamma.contiguous() if gamma is not None else empty, mean.contiguous(),
                         second.contiguous(), bool(is_meansq), float(eps), moving_mean if moving_mean is not None else empty,
                         moving_var if moving_var is not None else empty, float(momentum))


class _QBits(torch.autograd.Function):
    @staticmethod
    def forward(ctx, k, i, fb, kbi, add_mode):
        ctx.save_for_backward(i, fb)
        ctx.kbi = kbi
        return qbits_fwd(k, i, fb, kbi, add_mode)

    @staticmethod
    def backward(ctx, g):
        i, fb = ctx.saved_tensors
        di, dfb = qbits_bwd(g.contiguous(), i, fb, ctx.kbi)
        return None, (None if ctx.kbi else di), dfb, None, None


def qbits(k: Tensor, i, fb: Tensor, kbi: bool, add_mode: int = 0) -> Tensor:
    """Bit-widths ``relu(round(i) + round(f))`` (KIF) or ``round(b)`` (KBI) of raw quantizer variables, plus ``k``
    (``add_mode`` 1) or ``k * (b > 0)`` (``add_mode`` 2), with straight-through rounding; shaped like ``fb``."""
    empty = fb.new_empty(0)
    flush_tracks()
    return _QBits.apply(k if add_mode else empty, i if not kbi else empty, fb, bool(kbi), int(add_mode))


class _EbopsFinish(torch.autograd.Function):
    @staticmethod
    def forward(ctx, ebops, factor, beta, ebops_var):
        ctx.save_for_backward(beta)
        ctx.factor, ctx.shape = factor, ebops.shape
        return ebops_finish_fwd(ebops, factor, beta, ebops_var)

    @staticmethod
    def backward(ctx, g):
        (beta,) = ctx.saved_tensors
        return ebops_finish_bwd(g.contiguous(), beta, ctx.factor).view(ctx.shape), None, None, None


def ebops_finish(ebops: Tensor, factor: float, beta: Tensor, ebops_var: Tensor) -> Tensor:
    """``ebops * factor`` stored into the uint32 variable and returned times ``beta`` (the loss term)."""
    return _EbopsFinish.apply(ebops.contiguous(), float(factor), beta, ebops_var)


class _BitsEbops(torch.autograd.Function):
    """EBOPs that are algebra on bit-width tensors (``hgq_lut_ebops`` / ``hgq_sum_ebops`` / ``hgq_softmax_ebops`` / ``hgq_mha_ebops``).
    ``layouts[n]`` = ``(size, inner, kbi, add_mode)`` of operand n or ``None``; ``qvars`` = k, i, fb per operand
    (empty tensors where absent).  The kernel leaves the gradients for a unit upstream gradient; backward scales them."""

    @staticmethod
    def forward(ctx, kind, params, beta, ebops_var, layouts, owners, *qvars):
        ctx.owners = owners
        ks, is_, fbs = list(qvars[0::3]), list(qvars[1::3]), list(qvars[2::3])
        total = sum(2 * fb.numel() for fb, lay in zip(fbs, layouts) if lay is not None)
        buf = torch.empty(max(total, 1), dtype=torch.float32, device=beta.device)
        descs, slots, off = [], [], 0
        for k, i, fb, lay in zip(ks, is_, fbs, layouts):
            if lay is None:
                descs.append(None), slots.append(None)
                continue
            size, inner, kbi, add_mode = lay
            _check_f32('fb', fb)
            _need(fb.numel() == size and (kbi or i.numel() == size) and (not add_mode or k.numel() == size), 'operand sizes differ')
            n = fb.numel()
            g_i, g_fb = buf[off:off + n], buf[off + n:off + 2 * n]
            off += 2 * n
            slots.append((g_i, g_fb))
            descs.append(_lib.BitsDesc(k.data_ptr() if add_mode else None, None if kbi else i.data_ptr(), fb.data_ptr(), size, inner,
                                       int(kbi), int(add_mode), None if kbi else g_i.data_ptr(), g_fb.data_ptr()))
        out = torch.empty((), dtype=torch.float32, device=beta.device)
        if _DEFER['depth'] > 0 and _OVERLAP['depth'] > 0:
            # a step that runs its EBOPs launches beside the data kernels: this one goes out with the others when the
            # model call returns (outputs exist already; the integer bits it reads are guarded by `_reads_queued`)
            reads = {i.data_ptr() for i, lay in zip(is_, layouts) if lay is not None and not lay[2]}
            _keep(qvars + (out, buf))  # operands may be temporaries, outputs may be dropped: all outlive the launch on the second stream
            _DEFER['late'].append((reads, lambda: _BitsEbops._launch(kind, params, beta, ebops_var, descs, out)))
        else:
            flush_tracks()  # the bit-widths read here include integer bits whose update may still be queued
            _BitsEbops._launch(kind, params, beta, ebops_var, descs, out)
        ctx.save_for_backward(buf)
        ctx.slots = [None if s is None else (s[0].storage_offset(), s[1].storage_offset(), s[1].numel()) for s in slots]
        ctx.kbis = [None if lay is None else lay[2] for lay in layouts]
        ctx.shapes = [(i.shape, fb.shape) for i, fb in zip(is_, fbs)]
        ctx.mark_non_differentiable(ebops_var)
        return out

    @staticmethod
    def _launch(kind, params, beta, ebops_var, descs, out):
        lib = _lib.load()
        ptrs = [ctypes.addressof(d) if d is not None else None for d in descs]
        if kind == 'lut':
            n_cells, scale, factor = params
            rc = lib.hgq_lut_ebops(ptrs[0], ptrs[1], n_cells, scale, factor, _ptr(beta), _ptr(ebops_var), _ptr(out), _stream())
        elif kind == 'sum':
            n_cells, parallel_factor, n_parallel, factor = params
            rc = lib.hgq_sum_ebops(ptrs[0], n_cells, parallel_factor, n_parallel, factor, _ptr(beta), _ptr(ebops_var), _ptr(out), _stream())
        elif kind == 'softmax':
            rows, L, f1, f2 = params
            rc = lib.hgq_softmax_ebops(ptrs[0], ptrs[1], ptrs[2], rows, L, f1, f2, _ptr(beta), _ptr(ebops_var), _ptr(out), _stream())
        elif kind == 'conv':
            geom, F, conv_scale, bias_size, factor = params
            rc = lib.hgq_conv2d_ebops_q(ptrs[0], ptrs[1], ptrs[2], ctypes.byref(_geom(geom)), F, conv_scale, bias_size, factor, _ptr(beta),
                                        _ptr(ebops_var), _ptr(out), _stream())
        else:
            T, S, N, H, Hv, f1, f2 = params
            rc = lib.hgq_mha_ebops(ptrs[0], ptrs[1], ptrs[2], ptrs[3], T, S, N, H, Hv, f1, f2, _ptr(beta), _ptr(ebops_var), _ptr(out),
                                   _stream())
        _lib.check(rc, f'hgq_{kind}_ebops')

    @staticmethod
    def backward(ctx, g):
        (buf,) = ctx.saved_tensors
        n_args = 6 + 3 * len(ctx.slots)
        if _SINK['open'] and ctx.owners is not None:
            pieces = []
            for slot, kbi, own in zip(ctx.slots, ctx.kbis, ctx.owners):
                if slot is None:
                    continue
                oi, of, n = slot
                o_i, o_fb = own if own is not None else (None, None)
                pieces.append((o_fb, buf[of:of + n]))
                if not kbi and (o_i is None or o_i.requires_grad):  # an unknown owner makes the whole call fall back
                    pieces.append((o_i, buf[oi:oi + n]))
            if all(_parkable(o) for o, _ in pieces):
                for o, piece in pieces:
                    _stash_side(o, g, piece)
                return (None,) * n_args
        join_side()  # the kernel that fills `buf` may have run on the second stream
        scaled = buf if _is_unit(g) else buf * g  # one launch for every operand
        grads = [None, None, None, None, None, None]
        for slot, kbi, (i_shape, fb_shape) in zip(ctx.slots, ctx.kbis, ctx.shapes):
            if slot is None:
                grads += [None, None, None]
                continue
            oi, of, n = slot
            grads += [None, None if kbi else scaled[oi:oi + n].view(i_shape), scaled[of:of + n].view(fb_shape)]
        return tuple(grads)


class _BiasAddRows(torch.autograd.Function):
    """``y + b`` for a bias that spans (a broadcast of) one batch element.  The bias gradient, a sum over the batch, is
    taken by the library's fixed-order slice reduction: a framework reduction over many workgroups records a memory-clearing
    node when the step is captured in a graph, and such nodes have replayed wrongly on this platform."""

    @staticmethod
    def forward(ctx, y, b):
        ctx.b_shape = b.shape
        return y + b

    @staticmethod
    def backward(ctx, g):
        db = None
        if ctx.needs_input_grad[1]:
            g2 = g.contiguous().view(g.shape[0], -1)
            full = torch.empty(g2.shape[1], dtype=torch.float32, device=g.device)
            e = full.new_empty(0)
            reduce_slices_multi_op([g2], [full, e, e], [False, False, False])
            db = full.view(g.shape[1:]).sum_to_size(ctx.b_shape)  # over the bias' own broadcast axes, if any (small)
        return g, db


@torch.library.custom_op('hgq::affine_rows_fwd', mutates_args=())
def affine_rows_fwd(x: Tensor, s: Tensor, o: Tensor) -> Tensor:
    _check_f32('x', x), _check_f32('scale', s), _check_f32('offset', o)
    C = x.shape[-1]
    _need(s.numel() == C and o.numel() == C, 'scale and offset must have one entry per trailing channel')
    y = torch.empty_like(x)
    rc = _lib.load().hgq_affine_rows_fwd(_ptr(x), _ptr(s), _ptr(o), _ptr(y), x.numel() // C, C, _stream())
    _lib.check(rc, 'hgq_affine_rows_fwd')
    return y


@affine_rows_fwd.register_fake
def _(x, s, o):
    return torch.empty_like(x)


@torch.library.custom_op('hgq::affine_rows_bwd', mutates_args=())
def affine_rows_bwd(g: Tensor, x: Tensor, s: Tensor, need_dx: bool) -> tuple[Tensor, Tensor, Tensor]:
    _check_f32('g', g), _check_f32('x', x), _check_f32('scale', s)
    C = x.shape[-1]
    rows = x.numel() // C
    lib = _lib.load()
    dx = torch.empty_like(x) if need_dx else x.new_empty(0)
    ds, do = x.new_empty(C), x.new_empty(C)
    n_ws = lib.hgq_affine_rows_bwd_workspace(rows, C)
    _need(n_ws >= 0, 'hgq_affine_rows_bwd_workspace rejected the shape')
    ws = x.new_empty(max(int(n_ws), 1))
    rc = lib.hgq_affine_rows_bwd(_ptr(g), _ptr(x), _ptr(s), _ptr(dx), _ptr(ds), _ptr(do), _ptr(ws), rows, C, _stream())
    _lib.check(rc, 'hgq_affine_rows_bwd')
    return dx, ds, do


@affine_rows_bwd.register_fake
def _(g, x, s, need_dx):
    C = x.shape[-1]
    return (torch.empty_like(x) if need_dx else x.new_empty(0)), x.new_empty(C), x.new_empty(C)


class _AffineRows(torch.autograd.Function):
    """``x * s + o`` with ``s``, ``o`` of one value per trailing channel (a multiplication, then an addition, as the
    reference's ``inputs * qscale + qoffset``, src/hgq/layers/batch_normalization.py:184): one launch forward, and one
    pass + a fixed-order slice reduction backward for ``dx`` and the two sums over the rows."""

    @staticmethod
    def forward(ctx, x, s, o):
        ctx.save_for_backward(x, s)
        ctx.shapes = (s.shape, o.shape)
        return affine_rows_fwd(x, s.reshape(-1).contiguous(), o.reshape(-1).contiguous())

    @staticmethod
    def backward(ctx, g):
        x, s = ctx.saved_tensors
        dx, ds, do = affine_rows_bwd(g.contiguous(), x, s.reshape(-1).contiguous(), ctx.needs_input_grad[0])
        return (dx if ctx.needs_input_grad[0] else None, ds.view(ctx.shapes[0]) if ctx.needs_input_grad[1] else None,
                do.view(ctx.shapes[1]) if ctx.needs_input_grad[2] else None)


@torch.library.custom_op('hgq::quantizer_scale_div', mutates_args=())
def quantizer_scale_div_op(x: Tensor, scaler: float) -> Tensor:
    _check_f32('x', x)
    y = torch.empty_like(x)
    _lib.check(_lib.load().hgq_quantizer_scale_div(_ptr(x), _ptr(y), x.numel(), scaler, _stream()), 'hgq_quantizer_scale_div')
    return y


@quantizer_scale_div_op.register_fake
def _(x, scaler):
    return torch.empty_like(x)


@torch.library.custom_op('hgq::quantizer_tail_fwd', mutates_args=())
def quantizer_tail_fwd(q: Tensor, xs: Tensor, has_scaler: bool, scaler: float, has_noise: bool, noise: float, has_affine: bool, a0: float,
                       a1: float) -> Tensor:
    _check_f32('q', q)
    if has_noise:
        _check_f32('xs', xs)
        _need(xs.numel() == q.numel(), 'the quantizer\'s input and output must have the same size')
    out = torch.empty_like(q)
    rc = _lib.load().hgq_quantizer_tail_fwd(_ptr(q), _ptr(xs), _ptr(out), q.numel(), int(has_scaler), scaler, int(has_noise), noise,
                                            int(has_affine), a0, a1, _stream())
    _lib.check(rc, 'hgq_quantizer_tail_fwd')
    return out


@quantizer_tail_fwd.register_fake
def _(q, xs, has_scaler, scaler, has_noise, noise, has_affine, a0, a1):
    return torch.empty_like(q)


@torch.library.custom_op('hgq::quantizer_tail_bwd', mutates_args=())
def quantizer_tail_bwd(g: Tensor, has_scaler: bool, scaler: float, has_noise: bool, noise: float, has_affine: bool,
                       a0: float) -> tuple[Tensor, Tensor]:
    _check_f32('g', g)
    dq = torch.empty_like(g)
    dxs = torch.empty_like(g) if has_noise else g.new_empty(0)
    rc = _lib.load().hgq_quantizer_tail_bwd(_ptr(g), _ptr(dq), _ptr(dxs), g.numel(), int(has_scaler), scaler, int(has_noise), noise,
                                            int(has_affine), a0, _stream())
    _lib.check(rc, 'hgq_quantizer_tail_bwd')
    return dq, dxs


@quantizer_tail_bwd.register_fake
def _(g, has_scaler, scaler, has_noise, noise, has_affine, a0):
    return torch.empty_like(g), (torch.empty_like(g) if has_noise else g.new_empty(0))


class _ScaleDiv(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, scaler):
        ctx.scaler = scaler
        return quantizer_scale_div_op(x, scaler)

    @staticmethod
    def backward(ctx, g):
        return quantizer_scale_div_op(g.contiguous(), ctx.scaler), None


class _QuantizerTail(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, xs, scaler, noise, affine):
        ctx.args = (scaler is not None, float(scaler or 1.0), noise is not None, float(noise or 0.0), affine is not None,
                    float(affine[0]) if affine is not None else 1.0)
        return quantizer_tail_fwd(q, xs, *ctx.args, float(affine[1]) if affine is not None else 0.0)

    @staticmethod
    def backward(ctx, g):
        dq, dxs = quantizer_tail_bwd(g.contiguous(), *ctx.args)
        return dq, (dxs if ctx.args[2] and ctx.needs_input_grad[1] else None), None, None, None


def _wrapper_on_gpu(*tensors) -> bool:
    return all(t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and t.numel() > 0 for t in tensors)


def quantizer_scale_div(x: Tensor, scaler: float) -> Tensor:
    """``x / scaler`` as a true division (the first step of the reference's ``Quantizer.call``, src/hgq/quantizer/quantizer.py:50-51)."""
    if _wrapper_on_gpu(x):
        return _ScaleDiv.apply(x, float(scaler))
    return x / torch.full((), float(scaler), dtype=x.dtype, device=x.device)


def quantizer_tail(q: Tensor, xs: Tensor, scaler, noise, affine) -> Tensor:
    """What the reference's ``Quantizer.call`` does behind its internal quantizer (src/hgq/quantizer/quantizer.py:54-59):
    ``q * scaler``, the blend ``xs + noise * (. - xs)`` with the quantizer's input ``xs``, ``. * affine[0] + affine[1]`` -
    whichever of the three are not ``None`` - in one pass each way."""
    if scaler is None and noise is None and affine is None:
        return q
    if _wrapper_on_gpu(q, xs) and q.shape == xs.shape:
        return _QuantizerTail.apply(q, xs, scaler, noise, affine)
    out = q
    if scaler is not None:
        out = out * scaler
    if noise is not None:
        out = xs + noise * (out - xs)
    if affine is not None:
        out = out * affine[0] + affine[1]
    return out


@torch.library.custom_op('hgq::gdense_fwd', mutates_args=())
def gdense_fwd(x: Tensor, w: Tensor, bias: Tensor, act: int) -> Tensor:
    _check_f32('x', x), _check_f32('w', w)
    R, G, K = x.shape
    N = w.shape[2]
    _need(tuple(w.shape) == (G, K, N) and bias.numel() in (0, G * N), 'x [R, G, K], w [G, K, N], bias [G, N]')
    y = x.new_empty((R, G, N))
    rc = _lib.load().hgq_gdense_fwd(_ptr(x), _ptr(w), _ptr(bias), _ptr(y), R, G, K, N, act, _stream())
    _lib.check(rc, 'hgq_gdense_fwd')
    return y


@gdense_fwd.register_fake
def _(x, w, bias, act):
    return x.new_empty((x.shape[0], x.shape[1], w.shape[2]))


@torch.library.custom_op('hgq::gdense_bwd', mutates_args=())
def gdense_bwd(dy: Tensor, y: Tensor, x: Tensor, w: Tensor, has_bias: bool, act: int, need_dx: bool) -> tuple[Tensor, Tensor, Tensor]:
    _check_f32('dy', dy), _check_f32('x', x), _check_f32('w', w)
    R, G, K = x.shape
    N = w.shape[2]
    lib = _lib.load()
    dx = torch.empty_like(x) if need_dx else x.new_empty(0)
    dw = torch.empty_like(w)
    db = x.new_empty((G, N)) if has_bias else x.new_empty(0)
    n_ws = lib.hgq_gdense_bwd_workspace(R, G, K, N, int(has_bias))
    _need(n_ws >= 0, 'hgq_gdense_bwd_workspace rejected the shape')
    ws = x.new_empty(max(int(n_ws), 1))
    rc = lib.hgq_gdense_bwd(_ptr(dy), _ptr(y), _ptr(x), _ptr(w), _ptr(dx), _ptr(dw), _ptr(db), _ptr(ws), R, G, K, N, act, _stream())
    _lib.check(rc, 'hgq_gdense_bwd')
    return dx, dw, db


@gdense_bwd.register_fake
def _(dy, y, x, w, has_bias, act, need_dx):
    return (torch.empty_like(x) if need_dx else x.new_empty(0)), torch.empty_like(w), x.new_empty((x.shape[1], w.shape[2]) if has_bias else 0)


class _GDense(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w, bias, act):
        y = gdense_fwd(x, w, bias, act)
        ctx.save_for_backward(x, w, y)
        ctx.act, ctx.has_bias = act, bias.numel() > 0
        return y

    @staticmethod
    def backward(ctx, gy):
        x, w, y = ctx.saved_tensors
        dx, dw, db = gdense_bwd(gy.contiguous(), y, x, w, ctx.has_bias, ctx.act, ctx.needs_input_grad[0])
        return (dx if ctx.needs_input_grad[0] else None, dw if ctx.needs_input_grad[1] else None,
                db if (ctx.has_bias and ctx.needs_input_grad[2]) else None, None)


def gdense_supported(x3: Tensor, w3: Tensor) -> bool:
    return (x3.is_cuda and x3.dtype == torch.float32 and w3.dtype == torch.float32 and x3.dim() == 3 and w3.dim() == 3
            and bool(_lib.load().hgq_gdense_supported(x3.shape[0], x3.shape[1], x3.shape[2], w3.shape[2])))


def gdense(x3: Tensor, w3: Tensor, bias2, act: int = 0) -> Tensor:
    """``act(x3[r, g, :] @ w3[g] + bias2[g])`` for ``x3 [R, G, K]``, ``w3 [G, K, N]``, ``bias2 [G, N]`` or None."""
    b = bias2.contiguous() if bias2 is not None else x3.new_empty(0)
    return _GDense.apply(x3.contiguous(), w3.contiguous(), b, int(act))


def affine_rows(x: Tensor, s: Tensor, o: Tensor) -> Tensor:
    """``x * s + o`` for per-channel ``s`` and ``o`` along the last axis of ``x`` (any other layout: plain tensor operations)."""
    C = x.shape[-1] if x.dim() else 0
    if (x.is_cuda and x.dtype == torch.float32 and x.dim() >= 2 and x.numel() > 0 and s.numel() == C and o.numel() == C
            and s.shape[-1:] == (C,) and o.shape[-1:] == (C,) and s.dtype == torch.float32 and o.dtype == torch.float32
            and C % 4 == 0 and x.is_contiguous() and x.data_ptr() % 16 == 0):
        return _AffineRows.apply(x, s, o)
    return x * s + o


def bias_add_rows(y: Tensor, b: Tensor) -> Tensor:
    """``y + b`` with ``b`` broadcast over the leading (batch) axis of ``y`` only or also over trailing axes of size one."""
    bs = tuple(b.shape)
    if len(bs) == y.dim() and bs[0] == 1:
        bs = bs[1:]
    if (y.is_cuda and y.dtype == torch.float32 and b.dtype == torch.float32 and y.dim() >= 2 and y.shape[0] >= 1 and y.numel() > 0
            and len(bs) <= y.dim() - 1 and all(s in (1, t) for s, t in zip(reversed(bs), reversed(tuple(y.shape[1:]))))):
        return _BiasAddRows.apply(y, b)
    return y + b


def bits_ebops(kind: str, operands, params, beta: Tensor, ebops_var: Tensor, owners=None) -> Tensor:
    """Loss term ``ebops * beta`` of a layer whose EBOPs are algebra on bit-width tensors, in one launch; also assigns
    the uint32 variable.  ``operands``: per operand ``None`` or ``(k, i, fb, size, inner, kbi, add_mode)`` (``i`` is
    ``None`` for the (k, b, i) kind); ``params`` as the C entry point of ``kind`` ('lut', 'sum', 'softmax', 'mha', 'conv') takes them;
    ``owners``: per operand ``None`` or the variables ``(i, fb)`` behind it (see :class:`side_gradients`)."""
    e_f = beta.new_empty(0)
    e_k = torch.empty(0, dtype=torch.uint8, device=beta.device)
    if owners is None:  # operands that are the variables themselves own their gradient pieces
        as_var = lambda t: t if isinstance(t, torch.nn.Parameter) else None  # noqa: E731
        owners = [None if op is None else (as_var(op[1]), as_var(op[2])) for op in operands]
    flat, layouts = [], []
    for op in operands:
        if op is None:
            flat += [e_k, e_f, e_f]
            layouts.append(None)
            continue
        k, i, fb, size, inner, kbi, add_mode = op
        flat += [k if add_mode else e_k, e_f if kbi else i, fb]
        layouts.append((int(size), int(inner), bool(kbi), int(add_mode)))
    return _BitsEbops.apply(kind, tuple(params), beta, ebops_var, tuple(layouts), tuple(owners) if owners is not None else None, *flat)


class _AttnScores(torch.autograd.Function):
    @staticmethod
    def forward(ctx, query, key):
        ctx.save_for_backward(query, key)
        return attn_scores_fwd(query, key)

    @staticmethod
    def backward(ctx, g):
        query, key = ctx.saved_tensors
        return attn_scores_bwd(g.contiguous(), query, key)


class _AttnCombine(torch.autograd.Function):
    @staticmethod
    def forward(ctx, probs, value):
        ctx.save_for_backward(probs, value)
        return attn_combine_fwd(probs, value)

    @staticmethod
    def backward(ctx, g):
        probs, value = ctx.saved_tensors
        return attn_combine_bwd(g.contiguous(), probs, value)


def attn_scores(query: Tensor, key: Tensor) -> Tensor:
    """``einsum('aecd,abcd->acbe', key, query)``: query [B, T, N, H], key [B, S, N, H] -> [B, N, T, S]."""
    return _AttnScores.apply(query.contiguous(), key.contiguous())


def attn_combine(probs: Tensor, value: Tensor) -> Tensor:
    """``einsum('acbe,aecd->abcd', probs, value)``: probs [B, N, T, S], value [B, S, N, H] -> [B, T, N, H]."""
    return _AttnCombine.apply(probs.contiguous(), value.contiguous())


class _Pool2D(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, geom, is_max):
        ctx.save_for_backward(x)
        ctx.geom, ctx.is_max = tuple(geom), is_max
        return pool2d_fwd(x, list(geom), is_max)

    @staticmethod
    def backward(ctx, g):
        (x,) = ctx.saved_tensors
        return pool2d_bwd(g.contiguous(), x, list(ctx.geom), ctx.is_max), None, None


def pool2d(x: Tensor, pool_size, strides=None, padding: str = 'valid', mode: str = 'max') -> Tensor:
    """Max / average pooling of a channels-last [B, H, W, C] tensor; 'same' pads like Keras (odd pad after)."""
    B, H, W, C = x.shape
    ph, pw = pool_size
    sy, sx = strides if strides is not None else pool_size
    if padding == 'same':
        OH, OW = -(-H // sy), -(-W // sx)
        py, px = max((OH - 1) * sy + ph - H, 0) // 2, max((OW - 1) * sx + pw - W, 0) // 2
    else:
        OH, OW, py, px = (H - ph) // sy + 1, (W - pw) // sx + 1, 0, 0
    _need(OH >= 1 and OW >= 1, 'the pooling window does not fit the input')
    return _Pool2D.apply(x.contiguous(), (B, H, W, C, ph, pw, sy, sx, py, px, OH, OW), mode == 'max')


class _Conv2DEbops(torch.autograd.Function):
    @staticmethod
    def forward(ctx, bits_in, bits_ker, geom):
        total, g_in, g_ker = conv2d_ebops_op(bits_in, bits_ker, list(geom))
        ctx.save_for_backward(g_in, g_ker)
        return total

    @staticmethod
    def backward(ctx, g):
        g_in, g_ker = ctx.saved_tensors
        return g * g_in, g * g_ker, None


def conv_geometry(in_shape, kernel_shape, strides=(1, 1), padding='valid', dilation=(1, 1)):
    """The 14-entry geometry of a channels-last convolution; 'same' pads like Keras (odd pad after)."""
    B, H, W, C = in_shape
    kh, kw = kernel_shape[0], kernel_shape[1]
    (sy, sx), (dly, dlx) = strides, dilation
    eh, ew = dly * (kh - 1) + 1, dlx * (kw - 1) + 1
    if padding == 'same':
        OH, OW = -(-H // sy), -(-W // sx)
        py, px = max((OH - 1) * sy + eh - H, 0) // 2, max((OW - 1) * sx + ew - W, 0) // 2
    else:
        OH, OW, py, px = (H - eh) // sy + 1, (W - ew) // sx + 1, 0, 0
    _need(OH >= 1 and OW >= 1, 'the kernel does not fit the input')
    return (B, H, W, C, kh, kw, sy, sx, py, px, dly, dlx, OH, OW)


def conv2d_ebops(bits_in: Tensor, bits_ker: Tensor, strides=(1, 1), padding='valid', dilation=(1, 1)) -> Tensor:
    """``sum(conv2d(bits_in, bits_ker))`` for bit-width tensors [1, H, W, C] and [kh, kw, C, F], differentiable."""
    geom = conv_geometry(tuple(bits_in.shape), tuple(bits_ker.shape), strides, padding, dilation)
    return _Conv2DEbops.apply(bits_in.contiguous(), bits_ker.contiguous(), geom)


class _SparseCE(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, labels):
        loss, dlogits = sparse_ce_op(logits, labels)
        ctx.save_for_backward(dlogits)
        return loss

    @staticmethod
    def backward(ctx, g):
        (dlogits,) = ctx.saved_tensors
        return (dlogits if _is_unit(g) else g * dlogits), None


class _MSE(torch.autograd.Function):
    """With a gradient to come (``pred`` requires one), the forward pass also writes the gradient for a unit upstream
    gradient - one pass over the operands instead of two; another upstream gradient scales it."""

    @staticmethod
    def forward(ctx, pred, target):
        if pred.requires_grad:
            loss, dpred = mse_fwd_bwd_op(pred, target)
            ctx.save_for_backward(dpred)
            return loss
        ctx.save_for_backward()
        return mse_fwd_op(pred, target)

    @staticmethod
    def backward(ctx, g):
        (dpred,) = ctx.saved_tensors
        return (dpred if _is_unit(g) else g * dpred), None


def mse(pred: Tensor, target: Tensor | None = None) -> Tensor:
    """Mean squared error ``mean((pred - target) ** 2)``; ``target=None`` means zeros."""
    pred = pred.contiguous()
    if pred.numel() == 0:
        raise ValueError('mse of an empty tensor')
    return _MSE.apply(pred, target.contiguous() if target is not None else pred.new_empty(0))


@torch.library.custom_op('hgq::gather_batch', mutates_args=('state', 'x_dst', 'y_dst'))
def gather_batch(x_src: Tensor, y_src: Tensor, order: Tensor, state: Tensor, x_dst: Tensor, y_dst: Tensor) -> None:
    """The next batch of a data set in device memory: row r of ``x_dst`` / ``y_dst`` = row ``order[state[0] + r]`` of ``x_src`` /
    ``y_src``, and ``state[0]`` moves on by the batch size when the launch ends (``state``: two int64 words, zero when an epoch
    starts).  Recorded in a HIP graph the launch draws batch after batch as the graph is replayed."""
    n = x_src.shape[0]
    batch = x_dst.shape[0]
    for t in (x_src, y_src, x_dst, y_dst):
        _need(t.is_cuda and t.is_contiguous(), 'the data set and the batch buffers must be contiguous GPU tensors')
    _need(y_src.shape[0] == n and y_dst.shape[0] == batch and 1 <= batch <= n, 'samples and labels must agree in their first axis')
    _need(x_dst.dtype == x_src.dtype and y_dst.dtype == y_src.dtype and x_dst.shape[1:] == x_src.shape[1:] and y_dst.shape[1:] == y_src.shape[1:],
          'the batch buffers must have the data set\'s row shape and type')
    _need(order.dtype == torch.int64 and order.is_cuda and order.is_contiguous() and order.numel() == n, 'order must hold one int64 per row')
    _need(state.dtype == torch.int64 and state.is_cuda and state.numel() == 2, 'state must be two int64 words')
    xb, yb = x_src[0].numel() * x_src.element_size(), y_src[0].numel() * y_src.element_size()
    rc = _lib.load().hgq_gather_batch(_ptr(x_src), xb, _ptr(y_src), yb, _ptr(order), _ptr(state), _ptr(x_dst), _ptr(y_dst), batch, n, _stream())
    _lib.check(rc, 'hgq_gather_batch')


@gather_batch.register_fake
def _(x_src, y_src, order, state, x_dst, y_dst):
    return None


def sparse_ce(logits: Tensor, labels: Tensor) -> Tensor:
    """Mean sparse categorical cross-entropy from logits."""
    return _SparseCE.apply(logits.contiguous(), labels)


def sgd_update_(w, g, lr, l1=0.0, lo=float('-inf'), hi=float('inf')):
    sgd_update_op(w, g.contiguous(), float(lr), float(l1), float(lo), float(hi))


def sgd_update_multi_(ws, gs, l1, lo, hi, lr, sides=None, sum_terms=None, sum_out=None):
    """``gs[t]`` may be ``None``; ``sides[t]`` is a list of up to ``SGD_SIDES`` ``(scale or None, gradient)`` pairs.
    ``sum_terms`` / ``sum_out``: scalars added up in list order into ``sum_out`` by the update's launch."""
    n = len(ws)
    dev = ws[0].device
    empty = torch.empty(0, dtype=torch.float32, device=dev)
    flat_s, flat_c = [], []
    for t in range(n):
        pairs = list(sides[t]) if sides is not None else []
        if len(pairs) > SGD_SIDES:
            raise ValueError(f'at most {SGD_SIDES} side gradients per variable')
        for sc, sd in pairs:
            flat_s.append(sd.contiguous())
            flat_c.append(sc if sc is not None else empty)
        for _ in range(SGD_SIDES - len(pairs)):
            flat_s.append(empty), flat_c.append(empty)
    sgd_update_multi_op(list(ws), [g.contiguous() if g is not None else empty for g in gs], [float(v) for v in l1],
                        [float(v) for v in lo], [float(v) for v in hi], float(lr), flat_s, flat_c,
                        [t.detach() for t in sum_terms] if sum_terms else [], sum_out if sum_terms else empty)


# ======================================================================================
# gradient pieces that bypass autograd's accumulation
# ======================================================================================
# With the sink open, an EBOPs operator does not hand the gradients of the bit-width variables back to autograd (where
# each would cost a multiplication by the upstream gradient and an addition to the variable's other gradient, one
# library launch each): it leaves ``(upstream gradient, unit-upstream gradient)`` on the variable, and the optimizer's
# update kernel adds the pieces while it reads them.  Only an optimizer that consumes ``_hgq_side`` may open the sink.
_SINK = {'open': False, 'unit_ptr': 0, 'owners': None}


class side_gradients:
    """Context manager around ``loss.backward(root)``: opens the sink; ``root`` is the gradient the caller seeds the
    backward pass with when that gradient is exactly one (its address identifies "the upstream gradient is 1").
    ``owners``: the variables whose pieces the opening optimizer will consume (``id`` values); a piece for any other
    variable - one that another optimizer steps, or none - goes back to autograd instead of being parked where nobody
    reads it.  ``None`` accepts every variable."""

    def __init__(self, unit_root: Tensor | None = None, owners=None):
        self.unit_ptr = unit_root.data_ptr() if unit_root is not None else 0
        self.owners = owners

    def __enter__(self):
        _claim_step('side_gradients')
        self.prev = dict(_SINK)
        _SINK['open'], _SINK['unit_ptr'], _SINK['owners'] = True, self.unit_ptr, self.owners
        return self

    def __exit__(self, *exc):
        try:
            if exc[0] is None:
                flush_reductions()
            else:
                _PENDING_REDUCE.clear()
        finally:
            _SINK.update(self.prev)
            _release_step()


def _parkable(owner) -> bool:
    """A gradient piece for ``owner`` may be left with :func:`_stash_side`: the open sink's optimizer consumes it, or the
    variable is frozen and needs none.  (A trainable variable of another optimizer makes the caller fall back to autograd.)"""
    return owner is not None and (_sink_takes(owner) or not getattr(owner, 'requires_grad', False))


def _sink_takes(owner) -> bool:
    """The sink is open and ``owner`` is a trainable variable of the optimizer that opened it."""
    if owner is None or not _SINK['open'] or not getattr(owner, 'requires_grad', False):
        return False
    owners = _SINK['owners']
    return owners is None or id(owner) in owners


def _is_unit(g: Tensor) -> bool:
    """The tensor is (a view of) the seed gradient that the caller declared to be one."""
    return _SINK['unit_ptr'] != 0 and g.numel() == 1 and g.data_ptr() == _SINK['unit_ptr']


def _stash_side(owner, up, piece: Tensor) -> bool:
    """Leave ``up * piece`` (``up`` None: the piece as it is) on ``owner`` for the optimizer; False when the sink is
    closed or the owner is unknown."""
    if not _sink_takes(owner):
        return False
    if not hasattr(owner, '_hgq_side') or owner._hgq_side is None:
        owner._hgq_side = []
    owner._hgq_side.append((None if (up is None or _is_unit(up)) else up.reshape(1), piece.reshape(-1)))
    return True


def _owner(t):
    """The variable a kernel operand is (a view of), or None."""
    if isinstance(t, torch.nn.Parameter):
        return t
    base = getattr(t, '_base', None)
    return base if isinstance(base, torch.nn.Parameter) else None


def _can_route(owner, numel) -> bool:
    """``_route`` would leave a gradient of ``numel`` elements on ``owner`` rather than hand it back."""
    return _sink_takes(owner) and numel == owner.numel() and len(getattr(owner, '_hgq_side', None) or ()) < SGD_SIDES


def _route(owner, grad):
    """A finished gradient of a variable that also receives gradient from elsewhere: with the sink open it is left on
    the variable (returns None, so autograd has nothing to accumulate), otherwise handed back."""
    if grad is None or not _sink_takes(owner) or grad.numel() != owner.numel():
        return grad
    if len(getattr(owner, '_hgq_side', None) or ()) >= SGD_SIDES:
        return grad  # no room left in the update kernel's descriptor: autograd accumulates this one
    _stash_side(owner, None, grad.contiguous())
    return None


# ======================================================================================
# eager fast path
# ======================================================================================
# Every ``hgq::*`` operator above is registered with the dispatcher (fake tensors, tracing and ``torch.ops.hgq.*`` see
# it).  A call through the dispatcher costs the host some tens of microseconds - schema matching, the autograd and
# in-place bookkeeping layers the registration adds - which is several times the launch it wraps.  Inside this module the
# operators are only ever called from ``torch.autograd.Function`` bodies (no gradient mode, arguments already validated
# by the implementation itself), so when no dispatch mode is active the registered implementation is called directly.
def _direct(op):
    impl = op._init_fn

    def call(*args, **kwargs):
        if torch._C._len_torch_dispatch_stack() or torch.compiler.is_compiling():
            return op(*args, **kwargs)
        return impl(*args, **kwargs)

    call.__name__ = getattr(impl, '__name__', 'op')
    call.__doc__ = impl.__doc__
    call.op = op  # the dispatcher-registered operator
    call.register_fake = op.register_fake
    return call


def _install_direct_calls():
    from torch._library.custom_ops import CustomOpDef

    g = globals()
    for name, obj in list(g.items()):
        if isinstance(obj, CustomOpDef):
            g[name] = _direct(obj)


_install_direct_calls()
