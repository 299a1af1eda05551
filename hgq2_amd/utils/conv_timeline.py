"""Time line of the LDS-resident weight-gradient kernel's wavefronts (a measurement aid, not part of any compute path).

``make -C hgq2_amd/csrc prof`` builds ``libhgq_hip_prof.so``, in which workgroup 0 of ``wgrad_patch_kernel`` stamps the core
clock at its phase boundaries, one row of stamps per wavefront.  ``python -m hgq2_amd.utils.conv_timeline`` loads that build in
place of the product library, runs training steps of the image configuration (batch 1024, 28 x 28 x 1) and prints, per
wavefront, the median cycle count of every stamp since the workgroup started."""

import ctypes
import os
import statistics


def main(argv=None):
    from .. import _lib

    prof = os.path.join(os.path.dirname(_lib.LIB_PATH), 'libhgq_hip_prof.so')
    if not os.path.exists(prof):
        raise SystemExit(f'{prof} not found: run `make -C hgq2_amd/csrc prof`')
    _lib.LIB_PATH = prof
    import torch

    from .. import ops
    from ..train import SGD, model_loss
    from .models import conv_stack

    dev = torch.device('cuda:0')
    g = torch.Generator().manual_seed(0)
    torch.manual_seed(1)
    x = torch.rand(1024, 28, 28, 1, generator=g).to(dev)
    labels = torch.randint(0, 10, (1024,), generator=g).to(dev)
    model = conv_stack(device=dev)
    model(x, training=True)
    opt = SGD(model.parameters(), lr=1e-3, fold_regularizers=True)

    def step():
        opt.zero_grad()
        opt.backward(model_loss(model, ops.sparse_ce(model(x, training=True), labels), True))
        opt.step()

    for _ in range(5):
        step()
    torch.cuda.synchronize()
    lib = _lib.load()
    lib.hgq_wg_prof_read.restype = ctypes.c_int
    buf = (ctypes.c_ulonglong * 256)()
    runs = []
    for _ in range(9):
        step()
        torch.cuda.synchronize()
        if lib.hgq_wg_prof_read(buf) != 0:
            raise SystemExit('hgq_wg_prof_read failed')
        runs.append(list(buf))
    names = {0: 'start', 30: 'chains done', 31: 'end'}
    for it in range(3):
        names.update({1 + 8 * it: f'tile {it} top', 2 + 8 * it: f'tile {it} asked', 3 + 8 * it: f'tile {it} |B', 4 + 8 * it: f'tile {it} source stashed',
                      5 + 8 * it: f'tile {it} dz stashed', 6 + 8 * it: f'tile {it} |B'})
    for wave in (0, 1, 2):
        events = []
        for k, name in names.items():
            vals = [r[wave * 32 + k] - r[0] for r in runs if 0 <= r[wave * 32 + k] - r[0] < 10_000_000]
            if len(vals) >= 5:
                events.append((statistics.median(vals), name))
        events.sort()
        print(f'wave {wave} (cycles): ' + '  '.join(f'{name} {int(t)}' for t, name in events))
    return 0


if __name__ == '__main__':
    raise SystemExit(main())
