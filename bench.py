"""Benchmark: QDense MLP 16-64-32-32-5 training step at batch 16384 (samples/s), plus the
quantizer kernels' achieved HBM bandwidth on the 4 Mi-element standalone case, plus the CPU
oracle timed on the host cores as a baseline.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints one JSON line.  Everything is synthetic (seeded) data with inputs resident in HBM.
"""

from __future__ import annotations

import argparse
import contextlib
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E
# HBM bytes per launch of the 4 Mi-element quantizer kernels from rocprofv3 FETCH_SIZE / WRITE_SIZE
# counters, each scaled by what the same counter reads for the plain streaming kernel of known size
# (hgq_stream_probe); summary and commands in profiles/quantizer_4Mi_hbm_counters.md
TRAFFIC_BYTES = {'quant_fwd': 50.36e6, 'quant_bwd': 100.72e6, 'quant_fwd_sat': 83.88e6, 'quant_bwd_sat': 134.28e6,
                 'quant_fwd_bwd': 117.53e6, 'quant_fwd_bwd_sat': 151.07e6}
BATCH = 16384
DIMS = (16, 64, 32, 32, 5)
QN = 4 * 1024 * 1024  # standalone quantizer case: 4 Mi fp32 elements


def _cpu_threads():
    """Threads the CPU baseline runs on: the cores this process may use (its affinity mask; a GPU box hands a
    one-GPU job a share of the host, and OMP_NUM_THREADS names that share), not every core the host has."""
    try:
        allowed = len(os.sched_getaffinity(0))
    except AttributeError:
        allowed = os.cpu_count() or 1
    share = int(os.environ.get('OMP_NUM_THREADS', '0') or 0)
    return max(1, min(allowed, share) if share > 0 else allowed)


def _lib_bf16_parts():
    from hgq2_amd import _lib

    return bool(_lib.load().hgq_dense_use_bf16_parts(-1))


def _events_ms(fn, iters):
    import torch

    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / iters


def quantizer_roofline(iters=200):
    """Standalone KIF quantizer, RND rounding, per-element k, i, f, training forward + surrogate backward at 4 Mi
    elements, launched straight through the C ABI on torch's current stream and timed with HIP events on that stream.
    Two overflow modes: WRAP (the benchmark configuration; its training branch only rounds, so k and i never cross HBM)
    and SAT (every operand is live).  Next to them a plain streaming kernel (``hgq_stream_probe``) with the same number
    of bytes and a comparable read / write mix: what this memory system gives a kernel that does nothing else."""
    import torch

    from hgq2_amd import _lib

    lib = _lib.load()
    dev = torch.device('cuda:0')
    g = torch.Generator().manual_seed(0)
    # The MI355X has a 256 MB memory-side cache; one launch touches 50-134 MB, so re-running on
    # one buffer set would be served from that cache.  Rotate over enough distinct sets (> 1 GB in
    # total) that every launch streams from HBM.
    n_sets = 10
    sets = []
    for _ in range(n_sets):
        x = (torch.randn(QN, generator=g) * 2.0).to(dev)  # N(0, sigma^2 = 4)
        k = torch.ones(QN, device=dev)
        i = torch.randint(0, 5, (QN,), generator=g).float().to(dev)
        f = torch.randint(0, 9, (QN,), generator=g).float().to(dev)
        dy = torch.randn(QN, generator=g).to(dev)
        sets.append((x, k, i, f, dy) + tuple(torch.empty(QN, device=dev) for _ in range(4)))
    s = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731
    state = {'n': 0}

    def timed(fn, calls):
        # argument tuples are built once per buffer set: a launch is then one foreign call, so the host
        # keeps ahead of a 10-20 us kernel and the event-to-event time is kernel time
        def one():
            state['n'] += 1
            if fn(*calls[state['n'] % n_sets]):
                raise RuntimeError(lib.hgq_last_error().decode())

        for _ in range(10):
            one()
        return _events_ms(one, iters)

    out = {}
    for om in ('WRAP', 'SAT'):
        mode = _lib.mode_bits('RND', om, training=True)
        fwd_calls = [(p(x), p(k), p(i), p(f), p(y), None, None, QN, QN, 1, mode, s) for x, k, i, f, dy, y, dx, di, df in sets]
        bwd_calls = [(p(dy), p(x), p(k), p(i), p(f), p(dx), p(di), p(df), QN, QN, 1, mode, s) for x, k, i, f, dy, y, dx, di, df in sets]
        both_calls = [(p(x), p(k), p(i), p(f), p(dy), p(y), p(dx), p(di), p(df), QN, QN, 1, mode, s) for x, k, i, f, dy, y, dx, di, df in sets]
        t_fwd = timed(lib.hgq_quantize_fwd, fwd_calls)
        t_bwd = timed(lib.hgq_quantize_bwd, bwd_calls)
        t_both = timed(lib.hgq_quantize_fwd_bwd, both_calls)
        suffix = '' if om == 'WRAP' else '_sat'
        # operand bytes per element: forward x, k, i, f in, y out; backward dy, x, k, i, f in, dx, di, df out; both in one
        # launch x, k, i, f, dy in, y, dx, di, df out
        for name, ms, bpe in (('quant_fwd' + suffix, t_fwd, 20), ('quant_bwd' + suffix, t_bwd, 32), ('quant_fwd_bwd' + suffix, t_both, 36)):
            traffic = TRAFFIC_BYTES[name]
            out[name] = {'ms': ms, 'operand_bytes': bpe * QN, 'operand_GBps': bpe * QN / (ms * 1e-3) / 1e9,
                         'traffic': traffic, 'GBps': traffic / (ms * 1e-3) / 1e9, 'frac': traffic / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                         'frac_operands': bpe * QN / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
        out['quant_fwd_bwd' + suffix]['two_launches_ms'] = t_fwd + t_bwd
    # plain streaming kernels: 2 arrays read + 1 written (the bytes of the WRAP forward), 3 + 3 (the WRAP backward), 3 + 4 (both in one)
    for name, nr, nw in (('stream_2r1w', 2, 1), ('stream_3r3w', 3, 3), ('stream_3r4w', 3, 4), ('stream_1r1w', 1, 1)):
        calls = [(p(x), p(f), p(dy), p(y), p(dx), p(df), p(di), nr, nw, QN, s) for x, k, i, f, dy, y, dx, di, df in sets]
        ms = timed(lib.hgq_stream_probe, calls)
        nbytes = 4 * (nr + nw) * QN
        out[name] = {'ms': ms, 'traffic': nbytes, 'GBps': nbytes / (ms * 1e-3) / 1e9, 'frac': nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
    out['quant_fwd_bwd']['of_plain_stream'] = out['stream_3r4w']['ms'] / out['quant_fwd_bwd']['ms']
    out['quant_fwd']['of_plain_stream'] = out['stream_2r1w']['ms'] / out['quant_fwd']['ms']
    out['quant_bwd']['of_plain_stream'] = out['stream_3r3w']['ms'] / out['quant_bwd']['ms']
    return out


def softmax_roofline(iters=50, shape=(2048, 4, 64, 64), scaler=0.25):
    """Table softmax of the attention configuration (scores [2048, 4, 64, 64], 8-bit exp / inverse
    tables, per-position output quantizer): the one-pass kernels launched through the C ABI on
    torch's current stream, timed with HIP events on that stream.  Algorithmic bytes: forward
    8 B/element (scores in, probabilities out), backward 12 B/element (dy, scores in; dx out)."""
    import torch

    from hgq2_amd import _lib
    from hgq2_amd.config import LayerConfigScope, QuantizerConfig, QuantizerConfigScope
    from hgq2_amd.layers import QSoftmax

    lib = _lib.load()
    dev = torch.device('cuda:0')
    g = torch.Generator().manual_seed(0)
    with QuantizerConfigScope(place='all', default_q_type='kbi', overflow_mode='SAT_SYM'), \
            QuantizerConfigScope(place='datalane', default_q_type='kif', overflow_mode='WRAP'), \
            LayerConfigScope(enable_ebops=True, beta0=1e-5):
        layer = QSoftmax(axis=-1, enable_oq=True, input_scaler=scaler,
                         exp_iq_conf=QuantizerConfig(place='datalane', overflow_mode='SAT'))
    n_sets = 3  # 3 x (scores + output + dy + dx) = 1.6 GB: every launch streams from HBM
    sets = [tuple(torch.randn(shape, generator=g).to(dev) * (3.0 if j == 0 else 1.0) for j in range(2))
            + (torch.empty(shape, device=dev), torch.empty(shape, device=dev)) for _ in range(n_sets)]
    layer(sets[0][0], training=True)
    qs = layer._fused_plan(sets[0][0], True, None)
    assert qs is not None
    descs = [_lib.QDesc(q[0].data_ptr(), q[1].data_ptr(), q[2].data_ptr(), q[3] | _lib.MODE_K_U8) for q in qs]
    refs = [ctypes.addressof(d) for d in descs]
    L = shape[-1]
    n = 1
    for d in shape:
        n *= d
    rows, bw_rows = n // L, qs[4][1].numel() // L
    ws = torch.empty(lib.hgq_qsoftmax_bwd_workspace(rows, L, bw_rows, 1), device=dev)
    a1, a3 = (torch.empty(1, dtype=torch.int32, device=dev) for _ in range(2))
    ao = torch.empty(bw_rows * L, dtype=torch.int32, device=dev)
    gsh, goi, gof = torch.empty(8, device=dev), torch.empty(bw_rows * L, device=dev), torch.empty(bw_rows * L, device=dev)
    s = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731
    state = {'n': 0}

    def fwd():
        x, dy, y, dx = sets[state['n'] % n_sets]
        state['n'] += 1
        rc = lib.hgq_qsoftmax_fwd(p(x), p(y), rows, L, bw_rows, scaler, 1e-7, *refs, None, p(a3), p(ao), s)
        assert rc == 0

    def bwd():
        x, dy, y, dx = sets[state['n'] % n_sets]
        state['n'] += 1
        rc = lib.hgq_qsoftmax_bwd(p(dy), p(x), p(dx), rows, L, bw_rows, scaler, 1e-7, *refs, p(gsh), p(goi), p(gof), p(ws), s)
        assert rc == 0

    for _ in range(3):
        fwd(), bwd()
    out = {}
    for name, fn, bpe in (('qsoftmax_fwd', fwd, 8), ('qsoftmax_bwd', bwd, 12)):
        ms = _events_ms(fn, iters)
        gbs = bpe * n / (ms * 1e-3) / 1e9
        out[name] = {'ms': ms, 'bytes': bpe * n, 'GBps': gbs, 'frac': gbs / HBM_PEAK_GBS}
    return out


def dense_streaming(iters=20, rows=131072, K=64, N=64):
    """The streaming dense kernels (the contraction of QDense / QEinsumDense with the batch as rows) at rows x K x N with
    cold operands: six operand sets are rotated inside one captured HIP graph, timed with HIP events around its
    replays.  Run once per matrix instruction (fp32 `32x32x2`, and bf16 `32x32x16` on exact bf16 parts of the fp32
    operands) and per operand width (6 bits: one part; 12: two; 22: three).  Algorithmic bytes: forward
    4 (rows K + rows N) B; backward 4 (2 rows N + 2 rows K) B (dy, y, x in; dx out) plus the slices."""
    import torch

    from hgq2_amd import _lib, ops

    lib = _lib.load()
    dev = torch.device('cuda:0')
    g = torch.Generator().manual_seed(0)
    e = torch.empty(0, device=dev)
    n_sets = 6
    out = {}
    was = lib.hgq_dense_use_bf16_parts(-1)
    for bits in (6, 12, 22):
        xs = [(torch.round(torch.randn(rows, K, generator=g) * 2 ** (bits - 3)) / 2 ** (bits - 3)).to(dev) for _ in range(n_sets)]
        w = (torch.round(torch.randn(K, N, generator=g) * 2 ** (bits - 2)) / 2 ** bits).to(dev)
        b = torch.zeros(N, device=dev)
        dys = [torch.randn(rows, N, generator=g).to(dev) for _ in range(n_sets)]
        ys = [ops.qdense_fwd(x, e, e, e, w, b, 1, 0, 0, False)[0] for x in xs]
        for on, name in ((0, 'fp32'), (1, 'bf16_parts')):
            lib.hgq_dense_use_bf16_parts(on)
            for what, nbytes in (('fwd', 4 * rows * (K + N)), ('bwd', 8 * rows * (K + N))):
                def launches():
                    for x, dy, y in zip(xs, dys, ys):
                        if what == 'fwd':
                            ops.qdense_fwd(x, e, e, e, w, b, 1, 0, 0, False)
                        else:
                            ops.qdense_bwd(dy, y, x, e, w, True, 1, 0, 0)

                side = torch.cuda.Stream()
                side.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(side):
                    launches()
                torch.cuda.current_stream().wait_stream(side)
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=side):
                    launches()
                graph.replay()
                ms = _events_ms(graph.replay, iters) / n_sets
                gbs = nbytes / (ms * 1e-3) / 1e9
                out[f'{what}_{name}_{bits}bit'] = {'ms': ms, 'bytes': nbytes, 'GBps': gbs, 'frac': gbs / HBM_PEAK_GBS}
    lib.hgq_dense_use_bf16_parts(was)
    return out


def config_step_time(name, steps=20, warmup=5, graph=False, cpu=False, cpu_budget_s=15.0):
    """One training step (forward, backward, SGD update) of the configurations other than the headline one, at their full
    sizes: 'particle' (QEinsumDenseBatchnorm per-particle network, batch 4096 x 64 x 16), 'conv'
    (QConv2D stack on 28 x 28 x 1, batch 1024), 'mha' (QMultiHeadAttention, batch 2048 x 64 x 64)."""
    import torch

    from hgq2_amd import ops
    from hgq2_amd.train import SGD, model_loss
    from hgq2_amd.utils import models

    dev = torch.device('cuda:0')
    g = torch.Generator().manual_seed(0)
    torch.manual_seed(1)
    if name == 'particle':
        batch = 4096
        x = torch.randn(batch, 64, 16, generator=g).to(dev)
        labels = torch.randint(0, 5, (batch,), generator=g).to(dev)
        model = models.particle_mlp(device=dev)
        loss_fn = lambda out: ops.sparse_ce(out, labels)  # noqa: E731
    elif name == 'conv':
        batch = 1024
        x = torch.rand(batch, 28, 28, 1, generator=g).to(dev)
        labels = torch.randint(0, 10, (batch,), generator=g).to(dev)
        model = models.conv_stack(device=dev)
        loss_fn = lambda out: ops.sparse_ce(out, labels)  # noqa: E731
    elif name == 'mha':
        batch = 2048
        x = torch.randn(batch, 64, 64, generator=g).to(dev)
        model = models.mha_block(device=dev)
        labels = None
        loss_fn = lambda out: ops.mse(out) if out.is_cuda else (out * out).mean()  # noqa: E731
    else:
        raise ValueError(name)

    model(x, training=True)  # build
    opt = SGD(model.parameters(), lr=1e-3, fold_regularizers=True)

    def step():
        # forward, loss (+ EBOPs terms), backward, SGD update with the MonoL1 gradient and the
        # bit-width constraints folded into the update kernel
        with ops.overlap_ebops() if OVERLAP else contextlib.nullcontext():
            opt.zero_grad()
            loss = model_loss(model, loss_fn(model(x, training=True)), True)
            opt.backward(loss)
            opt.step()
        return loss.detach()

    run = step
    if graph:
        # the step is tens to hundreds of small launches: record it once, replay it
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        for p in model.parameters():
            p.grad = None
        g_ = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g_, stream=side):  # the stream of the warm-up steps: per-stream scratch made there is reused
            static_loss = step()

        def run():
            g_.replay()
            return static_loss

    for _ in range(warmup):
        run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        loss = run()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    out = {'workload': name, 'batch': batch, 'ms_per_step': ms, 'samples_per_s': batch / ms * 1e3, 'loss': float(loss),
           'launch': 'hip-graph replay' if graph else 'eager'}
    if cpu:
        out['cpu_baseline'] = _config_cpu_baseline(name, model, x, labels if name != 'mha' else None, batch, budget_s=cpu_budget_s)
        out['gpu_over_cpu'] = out['samples_per_s'] / out['cpu_baseline']['value']
    return out


def _config_cpu_baseline(name, model, x, labels, batch, budget_s=15.0):
    """The oracle's eager torch-CPU restatement of the same model (same weights and bit-widths) timed
    on the host cores: forward, loss, backward (no optimizer), a bounded number of steps."""
    import torch
    import torch.nn.functional as F

    from hgq2_amd.utils import models
    from oracle import twin

    cores = _cpu_threads()
    torch.set_num_threads(cores)
    xc = x.cpu()
    if name == 'mha':
        r = twin.ref_mha(model, tuple(xc.shape))

        def step():
            out = r(xc, training=True)
            ((out * out).mean() + r.extra_loss()).backward()
    else:
        twins = []
        shape = tuple(xc.shape)
        for layer in model.layers:
            if isinstance(layer, models.PARAMETER_FREE):
                twins.append(layer.host_fn)
                shape = tuple(layer.host_fn(torch.zeros(shape)).shape)
                continue
            kind = layer.__class__.__name__
            r = twin.ref_conv2d(layer) if kind == 'QConv2D' else (
                twin.ref_einsum_dense_bn(layer, shape) if kind == 'QEinsumDenseBatchnorm' else twin.ref_dense(layer))
            twins.append(r)
            shape = (shape[0],) + tuple(layer.compute_output_shape(shape)[1:])
        yc = labels.cpu()

        def step():
            h = xc
            extra = 0.0
            for t in twins:
                if callable(t) and not hasattr(t, 'extra_loss'):
                    h = t(h)
                else:
                    h = t(h, training=True)
                    extra = extra + t.extra_loss()
            (F.cross_entropy(h, yc) + extra).backward()

    step()
    n, t0 = 0, time.perf_counter()
    while True:
        step()
        n += 1
        el = time.perf_counter() - t0
        if el > budget_s or n >= 20:
            break
    return {'value': batch * n / el, 'unit': 'samples/s', 'cores': cores, 'host_cores': os.cpu_count(), 'kind': 'port',
            'sample': f'{n} forward+backward passes of the same model at batch {batch} (eager torch-CPU restatement of the reference path)'}


def cpu_baseline(budget_s=20.0):
    """The oracle's eager torch-CPU restatement of the reference path, same model and batch."""
    import torch

    from oracle import hgq_ref as ref

    cores = _cpu_threads()
    torch.set_num_threads(cores)
    g = torch.Generator().manual_seed(0)
    x = torch.randn(BATCH, DIMS[0], generator=g)
    labels = torch.randint(0, DIMS[-1], (BATCH,), generator=g)
    mlp = ref.RefMLP(dims=DIMS, seed=1)
    for _ in range(3):
        mlp.train_step(x, labels)
    n, t0 = 0, time.perf_counter()
    while True:
        mlp.train_step(x, labels)
        n += 1
        el = time.perf_counter() - t0
        if el > budget_s or n >= 200:
            break
    return {'value': BATCH * n / el, 'unit': 'samples/s', 'cores': cores, 'host_cores': os.cpu_count(), 'kind': 'port',
            'sample': f'{n} training steps of the same MLP at batch {BATCH} (eager torch-CPU restatement of the reference path)'}


OVERLAP = True  # EBOPs launches of the per-layer steps on a second stream (see hgq2_amd.ops.overlap_ebops)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=300)
    ap.add_argument('--warmup', type=int, default=30)
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--no-extras', action='store_true', help='headline and roofline only: skip the per-path and per-configuration timings')
    ap.add_argument('--roofline-only', action='store_true',
                    help='run only the standalone quantizer kernels and a plain copy of known size (for counter runs)')
    ap.add_argument('--config-step', choices=('particle', 'conv', 'mha'), default=None,
                    help='time one forward + backward pass of another configuration at full size instead of the headline run')
    ap.add_argument('--config-cpu', action='store_true', help='with --config-step: also time the CPU oracle of the same model')
    ap.add_argument('--no-overlap', action='store_true', help='keep the EBOPs launches of the per-layer steps on the main stream')
    ap.add_argument('--graph', action='store_true', help='with --config-step: capture the step in a HIP graph and replay it')
    ap.add_argument('--softmax-only', action='store_true',
                    help='run only the one-pass table-softmax kernels at the attention configuration (for profiler runs)')
    ap.add_argument('--dense-only', action='store_true',
                    help='run only the streaming dense kernels at 131072 x 64 x 64 with either matrix instruction (for profiler runs)')
    ap.add_argument('--path', choices=('fused', 'fused-graph', 'layers-graph', 'layers-eager'), default='fused',
                    help='fused: whole-step kernels (2 launches); layers: per-layer torch.library operators with autograd; '
                         '-graph: the step is captured once in a HIP graph and replayed')
    args = ap.parse_args()
    global OVERLAP
    OVERLAP = not args.no_overlap
    if args.gpus != 1:
        print(f'bench.py: this build runs on one GPU; --gpus {args.gpus} is not supported', file=sys.stderr)
        sys.exit(2)

    import torch

    if args.roofline_only:
        torch.cuda.set_device(0)
        print(json.dumps({'quantizer_kernels': quantizer_roofline(iters=50)}))
        return
    if args.config_step:
        torch.cuda.set_device(0)
        print(json.dumps({'config_step': config_step_time(args.config_step, steps=args.steps if args.steps != 300 else 20, graph=args.graph, cpu=args.config_cpu)}))
        return
    if args.softmax_only:
        torch.cuda.set_device(0)
        print(json.dumps({'softmax_kernels': softmax_roofline(iters=20)}))
        return

    if args.dense_only:
        torch.cuda.set_device(0)
        print(json.dumps({'dense_kernels': dense_streaming()}))
        return

    from hgq2_amd import ops
    from hgq2_amd.train import SGD, FusedQDenseStack, GraphedTrainStep, model_loss
    from hgq2_amd.utils.models import qdense_mlp

    dev = torch.device('cuda:0')
    torch.cuda.set_device(dev)
    g = torch.Generator().manual_seed(0)
    x = torch.randn(BATCH, DIMS[0], generator=g).to(dev)
    labels = torch.randint(0, DIMS[-1], (BATCH,), generator=g).to(dev)

    def make_step(path):
        """A fresh model (same seed) and one training step of it along `path`."""
        torch.manual_seed(1)
        model = qdense_mlp(DIMS, beta0=1e-5, device=dev)
        opt = SGD(model.parameters(), lr=0.01, fold_regularizers=True)
        if path == 'layers-eager':
            def step():
                opt.zero_grad()
                loss = model_loss(model, ops.sparse_ce(model(x, training=True), labels), True)
                opt.backward(loss)
                opt.step()
                return loss
            return step
        if path == 'layers-graph':
            return GraphedTrainStep(model, ops.sparse_ce, opt, x, labels, warmup=3)
        fused = FusedQDenseStack(model, lr=0.01)
        if path == 'fused':
            return lambda: fused.step(x, labels)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                fused.step(x, labels)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            fused.step(x, labels)

        def step():
            graph.replay()
            return fused.loss
        return step

    def time_steps(step, steps, warmup):
        for _ in range(warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            loss = step()
        torch.cuda.synchronize()
        return time.perf_counter() - t0, loss

    # the headline: exactly `steps` timed steps after `warmup` untimed ones
    step = make_step(args.path)
    el, loss = time_steps(step, args.steps, args.warmup)
    ms_per_step = el / args.steps * 1e3
    value = BATCH * args.steps / el

    labels_of = {'fused': 'whole-step kernels of a QDense stack with sparse CE and SGD, 2 launches (a special-case trainer)',
                 'fused-graph': 'the same whole-step kernels replayed from a HIP graph',
                 'layers-graph': 'the layer API: per-layer operators + autograd, the step replayed from a HIP graph',
                 'layers-eager': 'the layer API: per-layer operators + autograd, eager launches (host-bound)'}
    out = {
        'metric': 'QDense MLP train samples/s @bs16384; quantizer HBM GB/s vs peak',
        'value': value, 'unit': 'samples/s', 'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup,
        'ms_per_step': ms_per_step, 'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None, 'dtype': 'f32',
        'data': 'synthetic',
        'config': {'workload': 'QDense MLP 16-64-32-32-5 (ReLU hidden, linear out), batch 16384, kbi SAT_SYM weights, '
                               'kif WRAP datalanes, EBOPs beta0=1e-5, sparse CE, one fwd+bwd+SGD step; path = ' + args.path
                               + ': ' + labels_of[args.path]},
        'final_loss': float(loss),
        # which matrix instruction the contractions issued (results are the fp32 contraction either way: fp32 operands are
        # split exactly into bf16 parts, products exact in fp32, fp32 accumulation)
        'matrix_instruction': ('v_mfma_f32_32x32x16_bf16 on exact bf16 parts of the fp32 operands'
                               if _lib_bf16_parts() else 'v_mfma_f32_32x32x2_f32'),
        'batch_reuse': 'the same resident batch (1.1 MB) is fed every step: the step is latency-bound, its 6 MB working set '
                       'is served from cache',
    }
    if not args.no_extras:
        # every way the same step can be driven, each on a fresh model, over a few hundred steps
        paths = {}
        for path in ('fused', 'layers-graph', 'layers-eager'):
            n_steps = max(args.steps, 300 if path != 'layers-eager' else 100)
            el_p, _ = time_steps(make_step(path), n_steps, max(args.warmup, 10))
            paths[path.replace('-', '_')] = {'samples_per_s': BATCH * n_steps / el_p, 'ms_per_step': el_p / n_steps * 1e3, 'steps': n_steps,
                                             'what': labels_of[path]}
        # the epoch loop a user writes (hgq2_amd.train.fit: batches sliced from a resident data set, callbacks, the loss read
        # once per epoch), on the path it picks by itself and with the whole-step kernels switched off
        from hgq2_amd.train import fit
        n_batches = 64
        gx = torch.Generator().manual_seed(3)
        data_x = torch.randn(BATCH * n_batches, DIMS[0], generator=gx).to(dev)
        data_y = torch.randint(0, DIMS[-1], (BATCH * n_batches,), generator=gx).to(dev)
        for name, fused in (('fit_loop', None), ('fit_loop_layers', False)):
            torch.manual_seed(1)
            model = qdense_mlp(DIMS, beta0=1e-5, device=dev)
            fit(model, data_x, data_y, lr=0.01, batch_size=BATCH, epochs=1, shuffle=False, fused=fused)  # records / warms up
            times = {}
            for n_epochs in (5, 25):  # two lengths: their difference is steps only, the rest is the call's own set-up (the recording)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                hist = fit(model, data_x, data_y, lr=0.01, batch_size=BATCH, epochs=n_epochs, shuffle=False, fused=fused)
                torch.cuda.synchronize()
                times[n_epochs] = time.perf_counter() - t0
            per_step = (times[25] - times[5]) / (20 * n_batches)
            paths[name] = {'samples_per_s': BATCH / per_step, 'ms_per_step': per_step * 1e3, 'steps': 20 * n_batches,
                           'setup_ms_per_call': (times[5] - 5 * n_batches * per_step) * 1e3, 'final_epoch_loss': hist[-1]['loss'],
                           'what': 'train.fit over 64 resident batches: time per step from calls of 5 and 25 epochs (setup_ms_per_call = '
                                   'what a call takes beyond its steps: recording the step, reading the loss), '
                                   + ('path chosen by fit' if fused is None else 'per-layer operators replayed from a HIP graph')}
        out['paths'] = paths

    qr = quantizer_roofline()
    dom = qr['quant_fwd_bwd']
    out['roofline'] = {
        'bound': 'hbm', 'kernel': 'quant_fwd_bwd_pe<RND, WRAP>', 'achieved': dom['GBps'], 'peak': HBM_PEAK_GBS, 'unit': 'GB/s',
        'frac': dom['frac'], 'traffic': dom['traffic'], 'frac_operands': dom['frac_operands'],
        'of_plain_stream': dom['of_plain_stream'], 'two_launches_ms': dom['two_launches_ms'], 'ms': dom['ms'],
        'workload': 'standalone kif quantizer RND/WRAP, 4 Mi fp32 elements, per-element k/i/f: training forward + surrogate backward '
                    'in ONE launch (hgq_quantize_fwd_bwd).  achieved = HBM bytes per launch by the traffic counters (28 B/elem: x, f, '
                    'dy in; y, dx, di, df out - the WRAP training branch reads neither k nor i) / HIP-event time; frac_operands '
                    'prices the same time at all 36 B/elem of operands; of_plain_stream = time of a plain 3-read 4-write streaming '
                    'kernel of the same bytes / this kernel\'s time; two_launches_ms = hgq_quantize_fwd + hgq_quantize_bwd '
                    '(quantizer_kernels.quant_fwd / quant_bwd: the separate kernels priced the same way)'}
    sat = qr['quant_fwd_bwd_sat']
    out['roofline_all_operands_live'] = {
        'bound': 'hbm', 'kernel': 'quant_fwd_bwd_pe<RND, SAT>', 'achieved': sat['GBps'], 'peak': HBM_PEAK_GBS, 'unit': 'GB/s',
        'frac': sat['frac'], 'traffic': sat['traffic'], 'two_launches_ms': sat['two_launches_ms'], 'ms': sat['ms'],
        'workload': 'the same quantizer with overflow mode SAT: every operand is live, 36 B/elem cross HBM in the one-launch form '
                    '(separate launches: forward 20 B/elem, backward 32 B/elem, see quantizer_kernels.quant_fwd_sat / quant_bwd_sat)'}
    out['quantizer_kernels'] = qr
    if not args.no_cpu_baseline:
        out['cpu_baseline'] = cpu_baseline()
        out['gpu_over_cpu'] = value / out['cpu_baseline']['value']
        if 'paths' in out:
            for v in out['paths'].values():
                v['gpu_over_cpu'] = v['samples_per_s'] / out['cpu_baseline']['value']
    if not args.no_extras:
        # one training step of the other configurations at full size (HIP-graph replay), each with its CPU baseline
        out['config_steps'] = {name: config_step_time(name, steps=20, graph=True, cpu=not args.no_cpu_baseline, cpu_budget_s=6.0)
                               for name in ('particle', 'conv', 'mha')}
        # the streaming dense kernels alone, 131072 x 64 x 64 with cold operands, either matrix instruction
        out['dense_kernels'] = {k: {'ms': round(v['ms'], 5), 'GBps': round(v['GBps'], 1), 'frac': round(v['frac'], 4)}
                                for k, v in dense_streaming(iters=10).items()}
    print(json.dumps(out))


if __name__ == '__main__':
    main()
