"""Time line of the attention backward kernel's wavefronts (a measurement aid, not part of any compute path).

``make -C hgq2_amd/csrc prof`` builds ``libhgq_hip_prof.so``, in which workgroup 0 of ``qattn_bwd_kernel`` stamps the core
clock at every phase boundary of its first batch elements, one row of stamps per wavefront.  ``python -m
hgq2_amd.utils.attention_timeline`` loads that build in place of the product library, runs training steps of the attention
configuration (batch 2048, 64 x 64 tokens, 4 heads of 16) and prints, per wavefront and batch element, the median cycle
count of every stamp since the element's first one (the compiler may move work across a stamp: neighbouring phases trade a
few hundred cycles)."""

import ctypes
import os
import statistics

PHASES = ['top', '|B', 'stashed|B', 'scores+dprobs', 'exp fwd+sum', 'oq+probs', '|B', 'dv', 'exp bwd', 'dq', '|B', 'spill|B', 'dk']


def main(argv=None):
    from .. import _lib

    prof = os.path.join(os.path.dirname(_lib.LIB_PATH), 'libhgq_hip_prof.so')
    if not os.path.exists(prof):
        raise SystemExit(f'{prof} not found: run `make -C hgq2_amd/csrc prof`')
    _lib.LIB_PATH = prof
    import torch

    from .. import ops
    from ..train import SGD, model_loss
    from .models import mha_block

    dev = torch.device('cuda:0')
    torch.manual_seed(1)
    x = torch.randn(2048, 64, 64, generator=torch.Generator().manual_seed(0)).to(dev)
    model = mha_block(device=dev)
    model(x, training=True)
    opt = SGD(model.parameters(), lr=1e-3, fold_regularizers=True)

    def step():
        opt.zero_grad()
        opt.backward(model_loss(model, ops.mse(model(x, training=True)), True))
        opt.step()

    for _ in range(5):
        step()
    torch.cuda.synchronize()
    lib = _lib.load()
    lib.hgq_qa_prof_read.restype = ctypes.c_int
    buf = (ctypes.c_ulonglong * 512)()
    runs = []
    for _ in range(9):
        step()
        torch.cuda.synchronize()
        if lib.hgq_qa_prof_read(buf) != 0:
            raise SystemExit('hgq_qa_prof_read failed')
        runs.append(list(buf))
    for wave in (0, 1, 4, 7):
        for element in (1, 2):
            base = (wave * 4 + element) * 16
            at = [statistics.median(r[base + k] - r[base] for r in runs) for k in range(len(PHASES))]
            print(f'wave {wave} element {element} (cycles): ' + '  '.join(f'{n} {int(t)} (+{int(t - (at[k - 1] if k else 0))})' for k, (n, t) in enumerate(zip(PHASES, at))))
    return 0


if __name__ == '__main__':
    raise SystemExit(main())
