"""Time line of the whole-step QDense kernel's wavefronts (a measurement aid, not part of any compute path).

``make -C hgq2_amd/csrc prof`` builds ``libhgq_hip_prof.so``, in which workgroup 0 of ``mlp_fwd_bwd_kernel`` stamps the
100 MHz wall clock at every phase boundary, one row of stamps per wavefront.  ``python -m hgq2_amd.utils.mlp_timeline``
loads that build in place of the product library, runs steps of the benchmark stack (16-64-32-32-5, batch 16384) and
prints, per wavefront, the median time of every stamp in microseconds since the workgroup started."""

import ctypes
import os
import statistics
import sys

STAMPS = {0: 'start', 1: 'x asked', 2: 'image asked', 3: 'image in|B', 60: 'tile top', 61: 'stage loop', 32: 'staged', 4: '|B',
          33: 'fwd0', 5: '|B', 34: 'fwd1', 6: '|B', 35: 'fwd2', 7: '|B', 36: 'fwd3', 8: '|B', 16: 'loss|B',
          48: 'bwd3 dW chain', 52: 'bwd3 dW out', 56: 'bwd3 dx chain', 41: 'bwd3 done', 17: '|B',
          49: 'bwd2 dW chain', 53: 'bwd2 dW out', 57: 'bwd2 dx chain', 42: 'bwd2 done', 18: '|B',
          50: 'bwd1 dW chain', 54: 'bwd1 dW out', 58: 'bwd1 dx chain', 43: 'bwd1 done', 19: '|B',
          51: 'bwd0 dW chain', 55: 'bwd0 dW out', 59: 'bwd0 dx chain', 44: 'bwd0 done', 20: '|B', 30: 'tail', 31: 'flushed'}


def main(argv=None):
    from .. import _lib

    prof = os.path.join(os.path.dirname(_lib.LIB_PATH), 'libhgq_hip_prof.so')
    if not os.path.exists(prof):
        raise SystemExit(f'{prof} not found: run `make -C hgq2_amd/csrc prof`')
    _lib.LIB_PATH = prof
    import torch

    from ..train import FusedQDenseStack
    from .models import qdense_mlp

    dev = torch.device('cuda:0')
    g = torch.Generator().manual_seed(0)
    x = torch.randn(16384, 16, generator=g).to(dev)
    y = torch.randint(0, 5, (16384,), generator=g).to(dev)
    torch.manual_seed(1)
    stack = FusedQDenseStack(qdense_mlp((16, 64, 32, 32, 5), beta0=1e-5, device=dev), lr=0.01)
    for _ in range(20):
        stack.step(x, y)
    torch.cuda.synchronize()
    lib = _lib.load()
    lib.hgq_mlp_prof_read.restype = ctypes.c_int
    buf = (ctypes.c_ulonglong * 512)()
    runs = []
    for _ in range(11):
        stack.step(x, y)
        torch.cuda.synchronize()
        if lib.hgq_mlp_prof_read(buf) != 0:
            raise SystemExit('hgq_mlp_prof_read failed')
        runs.append(list(buf))
    for w in range(8):
        events = []
        for k, name in STAMPS.items():
            vals = [(r[w * 64 + k] - r[0]) / 100.0 for r in runs if 0 <= r[w * 64 + k] - r[0] < 10000]
            if len(vals) >= 6:
                events.append((statistics.median(vals), name))
        events.sort()
        print(f'wave {w}: ' + '  '.join(f'{name} {t:.2f}' for t, name in events))
    return 0


if __name__ == '__main__':
    sys.exit(main())
