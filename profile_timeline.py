#!/usr/bin/env python3
"""Where the life of a workgroup goes: a timeline of one launch of the Gated DeltaNet workgroup-per-key-head step or
of the KDA one-wavefront step.

    python -m statequant_amd.csrc.build --timeline        # once, here: writes statequant_amd/libsqhip_timeline.so
    python profile_timeline.py [--workload gdn-int8-g128 | kda-int4-g32] [--steps 3,7] [--out profiles]

The timeline library is the product library with marks compiled into `gdn_quad_kernel` (sq_gdn_quad.cuh) and
`kda_step_kernel` (sq_kda.cuh) by -DSQ_TIMELINE (sq_timeline.cuh): every wavefront stores the GPU's 100 MHz
real-time counter at 15 (KDA: 9) points of its life.  This script
builds bench.py's workload, runs whole fold periods back to back (eager launches, the 24 layer states in turn, as
bench.py does without a graph), and for each requested step of the fold period (0 .. m - 1; the last one folds) has
the last layer's launch of that step write its marks.  It prints and writes `<out>/<workload>_step_timeline.txt`:
the mean / median / 90th percentile of each interval over all wavefronts, the same per wavefront of the workgroup
(the wavefronts play different roles in the front end), workgroup starts and ends per 2 us and the number of resident
workgroups over the launch.  A mark costs a wavefront a wait for its scalar loads, about 0.08 us; a marked launch
runs about 10 % longer than the product's.
"""
from __future__ import annotations

import argparse
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import bench  # noqa: E402
from statequant_amd.kernels import _hip  # noqa: E402

MARKS_KDA = ['entry', 'slot known, token loads issued', 'fill count here, every load issued',
             'vectors, scales, buffered values staged', 'keys and decays here, coefficients done', 'state pass done',
             'outputs stored', 'appended', 'folded (full buffer), counters advanced']
MARKS = ['entry', 'item known (leading arguments here)', 'slot known, token loads issued', 'row blocks issued',
         'fill counter issued', 'fill count here, buffer loads issued', 'roles done, all loads landed in LDS',
         'first barrier passed', 'state pass done', 'buffer dot products done', 'second barrier passed',
         'output stored', 'largest |u| known (barrier)', 'appended, counters advanced', 'fold done and stored']
TICK_US = 0.01                                               # s_memrealtime counts at 100 MHz


def timeline(workload, step, dev, m=8):
    fam, bits, group, hv, hk, dk, dv, slots, layers = bench.WORKLOADS[workload]
    fam, lay, views, idx = bench.build(workload, m, dev)
    inputs, extra = bench.make_inputs(fam, lay, slots, layers, m, dev)
    out = torch.zeros(slots, hv, dv, device=dev, dtype=torch.bfloat16)
    waves = 4 if fam == 'gdn' else 1                         # GDN: two value heads x two wavefronts; KDA: one per head
    nwg = slots * hv // 2 if fam == 'gdn' else slots * hv
    buf = torch.zeros(nwg * waves * 16, dtype=torch.int64, device=dev)

    def run(s, upto):
        for L in range(upto):
            bench.launch(fam, lay, views[L], idx, inputs[s * layers + L], extra, out)

    for _ in range(4):                                       # warm up: states that have folded a few times
        for s in range(m):
            run(s, layers)
    for s in range(step):
        run(s, layers)
    run(step, layers - 1)
    os.environ['SQ_TIMELINE_BUF'] = f'{buf.data_ptr()}:{nwg * waves}'   # address : capacity in wavefronts, read at launch
    try:
        bench.launch(fam, lay, views[layers - 1], idx, inputs[step * layers + layers - 1], extra, out)
    finally:
        del os.environ['SQ_TIMELINE_BUF']
    torch.cuda.synchronize()
    t = buf.cpu().numpy().reshape(nwg, waves, 16)[:, :, :15].astype(np.float64)
    if not (t[:, :, 0] > 0).all():
        sys.exit(f'profile_timeline.py: {workload} did not run on an instrumented kernel (gdn_quad_kernel serves '
                 'Gated DeltaNet int4 / int8 states with key-axis groups, two value heads per key head; '
                 'kda_step_kernel every KDA state)')
    return t, nwg, fam


def report(workload, step, t, nwg, fam, m=8):
    marks = MARKS if fam == 'gdn' else MARKS_KDA
    last = (14 if step == m - 1 else 13) if fam == 'gdn' else 8
    waves = t.shape[1]
    T = (t - t[:, :, 0].min()) * TICK_US                     # us since the first wavefront started
    life = T[:, :, last] - T[:, :, 0]
    d = np.diff(T, axis=2)
    lines = [f'-- step {step} of the fold period ({"the fold step" if step == m - 1 else "a plain step"}), '
             f'{nwg} workgroups of {waves} wavefront{"s" if waves > 1 else ""} --',
             f'launch: first wavefront starts at 0, last one ends at {T[:, :, :last + 1].max():.2f} us',
             f'wavefront life, us: mean {life.mean():.2f}  median {np.median(life):.2f}  10 % {np.percentile(life, 10):.2f}'
             f'  90 % {np.percentile(life, 90):.2f}',
             'interval, us over all wavefronts:                                                 mean  median   90 %']
    for k in range(last):
        lines.append(f'  {marks[k]:<38} -> {marks[k + 1]:<38} {d[:, :, k].mean():6.2f} {np.median(d[:, :, k]):6.2f} '
                     f'{np.percentile(d[:, :, k], 90):6.2f}')
    first = T[:, 0, 0] < 1.0                                 # workgroups that the launch starts with
    if first.any() and not first.all():
        lines.append(f'mean of each interval, the {int(first.sum())} workgroups resident from the start / the others:')
        lines.append('  from the start: ' + ' '.join(f'{d[first][:, :, k].mean():5.2f}' for k in range(last)))
        lines.append('  the others:     ' + ' '.join(f'{d[~first][:, :, k].mean():5.2f}' for k in range(last)))
    if waves > 1:
        lines.append('mean of each interval by wavefront of the workgroup (1 and 3: q and k vectors; 0 and 2: gates; '
                     '2: key append):')
        for w in range(waves):
            lines.append(f'  wavefront {w}: ' + ' '.join(f'{d[:, w, k].mean():5.2f}' for k in range(last)))
    st, en = T[:, 0, 0], T[:, :, last].max(axis=1)
    edges = np.arange(0, T[:, :, :last + 1].max() + 2, 2.0)
    lines.append('workgroups starting per 2 us: ' + ' '.join(str(x) for x in np.histogram(st, edges)[0]))
    lines.append('workgroups ending per 2 us:   ' + ' '.join(str(x) for x in np.histogram(en, edges)[0]))
    lines.append('resident workgroups at t us:  ' + ' '.join(f'{x:.0f}:{int(((st <= x) & (en > x)).sum())}'
                                                            for x in np.arange(1, T[:, :, :last + 1].max(), 2.0)))
    if fam == 'gdn':                                         # when the row blocks are asked for and when they are all here
        e1 = np.arange(0, T[:, :, :last + 1].max() + 1, 1.0)
        lines.append('wavefronts asking for their row blocks per 1 us: ' + ' '.join(str(x) for x in np.histogram(T[:, :, 3], e1)[0]))
        lines.append('wavefronts with every load landed per 1 us:      ' + ' '.join(str(x) for x in np.histogram(T[:, :, 6], e1)[0]))
    return lines


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--workload', default='gdn-int8-g128', choices=sorted(bench.WORKLOADS))
    ap.add_argument('--steps', default='3,7', help='steps of the fold period to mark (the last one, m - 1, folds)')
    ap.add_argument('--out', default='profiles')
    a = ap.parse_args()
    lib = os.path.join(os.path.dirname(_hip.LIB_PATH), 'libsqhip_timeline.so')
    if not os.path.exists(lib):
        sys.exit(f'profile_timeline.py: {lib} is missing; build it with `python -m statequant_amd.csrc.build --timeline`')
    _hip.LIB_PATH = lib
    if not torch.cuda.is_available():
        sys.exit('profile_timeline.py: no GPU visible')
    if bench.WORKLOADS[a.workload][0] not in ('gdn', 'kda'):
        sys.exit('profile_timeline.py: only the Gated DeltaNet workgroup-per-key-head kernel and the KDA kernel carry '
                 'the marks')
    dev = torch.device('cuda:0')
    torch.cuda.set_device(dev)
    lines = [f'timeline of the decode-step kernel, bench.py workload {a.workload}',
             f'made by: python -m statequant_amd.csrc.build --timeline && python profile_timeline.py --workload '
             f'{a.workload} --steps {a.steps}',
             'marks: s_memrealtime (100 MHz) in every wavefront of one launch, the last of 24 back-to-back layer '
             'launches of the step; a marked launch runs about 10 % longer than the product kernel', '']
    for step in (int(x) for x in a.steps.split(',')):
        t, nwg, fam = timeline(a.workload, step, dev)
        lines += report(a.workload, step, t, nwg, fam) + ['']
    text = '\n'.join(lines)
    print(text)
    os.makedirs(a.out, exist_ok=True)
    path = os.path.join(a.out, f'{a.workload}_step_timeline.txt')
    with open(path, 'w') as f:
        f.write(text)
    print(f'wrote {path}')


if __name__ == '__main__':
    main()
