"""Time line of the streaming dense kernels' wavefronts (a measurement aid, not part of any compute path).

``make -C hgq2_amd/csrc prof`` builds ``libhgq_hip_prof.so``, in which workgroup 0 of ``qdense_fwd_bf16_kernel``, of
``qdense_bwd_fast_kernel`` and of ``dense_moments_bwd_gram_kernel`` stamps the constant-rate counter (10 ns ticks) at its phase
boundaries, one row of stamps per wavefront.  ``python -m hgq2_amd.utils.dense_timeline [rows K N]`` loads that build in place
of the product library, runs ``hgq_qdense_fwd``, ``hgq_qdense_bwd`` and ``hgq_qdense_moments_bwd`` on synthetic operands (a per-column input quantizer, an 8-bit kernel, default
131072 x 64 x 64: a projection of the attention configuration) and prints the median time of every stamp since the
workgroup started, for the first wavefront of each kernel."""

import ctypes
import os
import statistics
import sys


def main(argv=None):
    from .. import _lib

    prof = os.path.join(os.path.dirname(_lib.LIB_PATH), 'libhgq_hip_prof.so')
    if not os.path.exists(prof):
        raise SystemExit(f'{prof} not found: run `make -C hgq2_amd/csrc prof`')
    _lib.LIB_PATH = prof
    import torch

    args = list(sys.argv[1:] if argv is None else argv)
    rows, K, N = (int(a) for a in args[:3]) if len(args) >= 3 else (131072, 64, 64)
    dev = torch.device('cuda:0')
    g = torch.Generator().manual_seed(0)
    x = torch.randn(rows, K, generator=g).to(dev)
    dy = torch.randn(rows, N, generator=g).to(dev)
    w = (torch.randn(K, N, generator=g) * 8).round().div(16).to(dev)
    k_in, i_in, f_in = torch.ones(K, device=dev), torch.full((K,), 3.0, device=dev), torch.full((K,), 4.0, device=dev)
    lib = _lib.load()
    lib.hgq_db_prof_read.restype = ctypes.c_int
    mode = _lib.mode_bits('RND', 'WRAP', training=True)
    y, dx = torch.empty(rows, N, device=dev), torch.empty_like(x)
    amax = torch.empty(lib.hgq_qdense_fwd_parts(rows) * K, dtype=torch.int32, device=dev)
    ws = torch.empty(lib.hgq_qdense_bwd_workspace(rows, K, N, 1), dtype=torch.float32, device=dev)
    dqw, dqb, df = torch.empty(K, N, device=dev), torch.empty(N, device=dev), torch.empty(K, device=dev)
    gm, gsq, dy_in = torch.randn(N, generator=g).to(dev), torch.randn(N, generator=g).to(dev), torch.randn(rows, K, generator=g).to(dev)

    def run():
        rc = lib.hgq_qdense_fwd(x.data_ptr(), k_in.data_ptr(), i_in.data_ptr(), f_in.data_ptr(), 1, w.data_ptr(), None, y.data_ptr(),
                                amax.data_ptr(), rows, K, N, 0, mode, None)
        _lib.check(rc, 'hgq_qdense_fwd')
        rc = lib.hgq_qdense_bwd(dy.data_ptr(), None, x.data_ptr(), f_in.data_ptr(), 1, w.data_ptr(), dx.data_ptr(), dqw.data_ptr(),
                                dqb.data_ptr(), df.data_ptr(), ws.data_ptr(), rows, K, N, 0, mode, None)
        _lib.check(rc, 'hgq_qdense_bwd')
        if K % 4 == 0 and N % 4 == 0:  # (the statistics' backward takes no other widths)
            rc = lib.hgq_qdense_moments_bwd(x.data_ptr(), f_in.data_ptr(), 1, mode, w.data_ptr(), gm.data_ptr(), gsq.data_ptr(), dy_in.data_ptr(),
                                            dx.data_ptr(), dqw.data_ptr(), df.data_ptr(), ws.data_ptr(), rows, K, N, None)
            _lib.check(rc, 'hgq_qdense_moments_bwd')

    for _ in range(3):
        run()
    torch.cuda.synchronize()
    buf = (ctypes.c_ulonglong * 384)()
    runs = []
    for _ in range(9):
        run()
        torch.cuda.synchronize()
        if lib.hgq_db_prof_read(buf) != 0:
            raise SystemExit('hgq_db_prof_read failed')
        runs.append(list(buf))
    fwd = {0: 'start', 1: 'kernel matrix, bit-widths, LDS cleared, first tile in', 30: 'tiles done', 31: 'end'}
    bwd = dict(fwd)
    stats = {0: 'start', 1: 'kernel matrix, A and v, bit-widths, first tile in', 30: 'tiles done', 31: 'end'}
    for it in range(4):
        fwd.update({2 + 6 * it: f'tile {it} staged', 3 + 6 * it: f'tile {it} |barrier', 4 + 6 * it: f'tile {it} matrix instructions',
                    5 + 6 * it: f'tile {it} result in LDS', 6 + 6 * it: f'tile {it} |barrier'})
        bwd.update({2 + 6 * it: f'tile {it} top |barrier', 3 + 6 * it: f'tile {it} staged', 4 + 6 * it: f'tile {it} |barrier',
                    5 + 6 * it: f'tile {it} matrix instructions', 6 + 6 * it: f'tile {it} |barrier', 7 + 6 * it: f'tile {it} dx in LDS |barrier'})
        stats.update({2 + 6 * it: f'tile {it} top |barrier', 3 + 6 * it: f'tile {it} staged', 4 + 6 * it: f'tile {it} |barrier',
                      5 + 6 * it: f'tile {it} matrix instructions', 6 + 6 * it: f'tile {it} |barrier', 7 + 6 * it: f'tile {it} dx in LDS |barrier'})
    print(f'rows {rows}, K {K}, N {N}; microseconds since the start of workgroup 0, wavefront 0')
    for kernel, names in (('forward', fwd), ('backward', bwd), ('statistics', stats)):
        base = {'forward': 0, 'backward': 4 * 32, 'statistics': 8 * 32}[kernel]
        for k in sorted(names):
            vals = [r[base + k] - r[base] for r in runs if 0 <= r[base + k] - r[base] < 10_000_000]
            if vals and (k == 0 or statistics.median(vals) > 0):
                print(f'  {kernel:10s} {names[k]:55s} {statistics.median(vals) / 100:8.2f}')


if __name__ == '__main__':
    main()
